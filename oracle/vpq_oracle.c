/*
 * vpq_oracle.c -- CPU restatement of VPIPE's 4-bit / group-64 affine
 * quantized matmul path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against and the timed CPU baseline of the benchmark.  Nothing in
 * the shipped library links, loads or calls it.
 *
 * Every function cites the file:line of the reference (tgo-app-dev/vpipe) it
 * restates.  Paths are relative to the reference tree.  The reference's own
 * implementation is Metal Shading Language + Objective-C++ and cannot be built
 * on Linux, so nothing here is compiled from it; the algorithms are restated.
 *
 * What pins each function (checked in tests/test_oracle_*.py):
 *   bf16/f16 conversions   exhaustive agreement with torch / numpy casts
 *   dequant                numpy re-derivation from the three independent
 *                          layout statements in the reference + closed forms
 *   qmv / qmm              one-hot activations (y == W[n,k]), degenerate
 *                          quantizers (q=0, b=-8s&q=8, s=0), float64 numpy
 *                          matmul, linearity, the reference tests' own
 *                          procedural inputs and asserted tolerances
 *   lora                   float64 numpy, scale 0 == no adapter, the
 *                          reference's M=96 test shape (reduced) tolerance
 *   swiglu / interleave    x*expit(x) of scipy, silu(v) - silu(-v) == v, limits;
 *                          numpy stacking; fused pack == silu(qmv(gate)) * qmv(up)
 *                          from two separate packs
 *   w8g64                  numpy re-derivation from the byte view of the words, one-hot
 *                          activations, float64 matmul
 *   quantize (packer)      exact recovery of on-grid data, the reference's
 *                          round-trip error bounds, numpy re-derivation
 *   requantizer (8 -> 4)   bytes 17 c requantize to the nibbles c in k order (byte / nibble
 *                          order, word layout), constant group, codes 0 and 15 used in every
 *                          group, half-step reconstruction bound, vectorized numpy statement
 *                          (the last bit of Metal's fast division is not pinned)
 * Parity that only an Apple-GPU run could pin -- the last-bit effect of the
 * Metal kernels' summation order (simd_sum tree, steel BlockMMA K order,
 * matmul2d) -- is NOT pinned: the oracle accumulates in double instead, and
 * kernels are compared to it within the stated tolerance.
 *
 * Packed layout (gpu-kernels/metal/quant/affine_dequant.metal:45-52,
 * affine_qmm_mma.metal:98-99, tests/unit-tests/metal-lm/quant-gemv.cc:245-248):
 *   w       uint32 [N, K/8]   q[n, 8j+i] = (w[n,j] >> 4i) & 0xF
 *   scales  elt    [N, K/64]
 *   biases  elt    [N, K/64]  W[n,k] = scales[n,k/64]*q[n,k] + biases[n,k/64]
 * Element type is bf16 carried as uint16_t.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define VPO_GROUP 64

/* ---- scalar conversions ------------------------------------------------ */

/* tests/unit-tests/metal-compute-gemm-mma.cc:41-46 (round to nearest even on
 * the upper 16 bits).  NaN is kept a NaN, which the reference helper does not
 * guarantee; no test input contains one. */
uint16_t vpo_f32_to_bf16(float f)
{
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) { return (uint16_t)((x >> 16) | 0x40u); }
  const uint32_t rounding = 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)((x + rounding) >> 16);
}

/* tests/unit-tests/metal-compute-gemm-mma.cc:47-52 */
float vpo_bf16_to_f32(uint16_t h)
{
  const uint32_t x = (uint32_t)h << 16;
  float f;
  memcpy(&f, &x, 4);
  return f;
}

/* IEEE binary16 <-> binary32, round to nearest even.  The packer emits its
 * scales and biases with Metal's `(half)` cast
 * (gpu-kernels/metal/quant/affine_dequant.metal:270-271), which is this. */
uint16_t vpo_f32_to_f16(float f)
{
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t ax = x & 0x7fffffffu;
  if (ax > 0x7f800000u) { return (uint16_t)(sign | 0x7e00u); }       /* NaN */
  if (ax >= 0x47800000u) { return (uint16_t)(sign | 0x7c00u); }      /* >= 65536: inf */
  if (ax < 0x33000000u) { return (uint16_t)sign; }                   /* < 2^-25 */
  int e = (int)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u;                         /* 24-bit */
  int shift;                                                         /* bits to drop */
  uint32_t base;
  if (e < -14) { shift = 13 + (-14 - e); base = 0; }                 /* subnormal */
  else         { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
  const uint32_t keep = m >> shift;
  const uint32_t rem = m & ((1u << shift) - 1u);
  const uint32_t half = 1u << (shift - 1);
  uint32_t h = base + keep;
  if (rem > half || (rem == half && (keep & 1u))) { h += 1; }        /* carries into exp */
  return (uint16_t)(sign | h);
}

float vpo_f16_to_f32(uint16_t h)
{
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1fu;
  const uint32_t m = h & 0x3ffu;
  uint32_t x;
  if (e == 0) {
    if (m == 0) { x = sign; }
    else {
      float v = (float)m * 5.9604644775390625e-8f;                   /* m * 2^-24 */
      memcpy(&x, &v, 4);
      x |= sign;
    }
  } else if (e == 31) { x = sign | 0x7f800000u | (m << 13); }
  else { x = sign | ((e + 112u) << 23) | (m << 13); }
  float f;
  memcpy(&f, &x, 4);
  return f;
}

/* Loaders of bf16 models turn the packer's F16 scales/biases into bf16 once at
 * load (docs/PLUGINS.md:210-213,
 * generative-models/minimax-h3/metal-minimax-h3-transformer.cc:766-778). */
void vpo_f16_to_bf16_array(const uint16_t* in, uint16_t* out, size_t n)
{
  for (size_t i = 0; i < n; ++i) { out[i] = vpo_f32_to_bf16(vpo_f16_to_f32(in[i])); }
}

void vpo_f32_to_bf16_array(const float* in, uint16_t* out, size_t n)
{
  for (size_t i = 0; i < n; ++i) { out[i] = vpo_f32_to_bf16(in[i]); }
}

void vpo_f32_to_f16_array(const float* in, uint16_t* out, size_t n)
{
  for (size_t i = 0; i < n; ++i) { out[i] = vpo_f32_to_f16(in[i]); }
}

void vpo_f16_to_f32_array(const uint16_t* in, float* out, size_t n)
{
  for (size_t i = 0; i < n; ++i) { out[i] = vpo_f16_to_f32(in[i]); }
}

static inline unsigned code8(const uint32_t* w, size_t n, int Kw, int k);
static inline unsigned nibble(const uint32_t* w, size_t n, int Kw, int k)
{
  return (w[n * (size_t)Kw + (size_t)(k >> 3)] >> (4 * (k & 7))) & 0xfu;
}

/* ---- a1: dequant ------------------------------------------------------- */

/* gpu-kernels/metal/quant/affine_dequant.metal:25-58: one u32 word -> eight
 * outputs, out = (elt)(s * (float)q + b) with s, b widened to fp32.  s*q is
 * exact in fp32 (8-bit x 4-bit significands) so a fused or unfused multiply-add
 * gives the same fp32 value; it is written as two operations here and compiled
 * with -ffp-contract=off. */
void vpo_dequant_w4g64_f32(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           float* out, int K, int N)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_bf16_to_f32(scales[n * Kg + k / VPO_GROUP]);
      const float b = vpo_bf16_to_f32(biases[n * Kg + k / VPO_GROUP]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      out[n * (size_t)K + k] = sq + b;
    }
  }
}

void vpo_dequant_w4g64_bf16(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            uint16_t* out, int K, int N)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_bf16_to_f32(scales[n * Kg + k / VPO_GROUP]);
      const float b = vpo_bf16_to_f32(biases[n * Kg + k / VPO_GROUP]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      out[n * (size_t)K + k] = vpo_f32_to_bf16(sq + b);
    }
  }
}

/* group-32 twin, gpu-kernels/metal/quant/affine_dequant.metal:196-228 (GGUF Q4_0 repacked to
 * affine): the same expression with a scale and a bias per 32 values, scales/biases [N, K/32]. */
void vpo_dequant_w4g32_bf16(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            uint16_t* out, int K, int N)
{
  const int Kw = K / 8, Kg = K / 32;
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_bf16_to_f32(scales[n * Kg + k / 32]);
      const float b = vpo_bf16_to_f32(biases[n * Kg + k / 32]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      out[n * (size_t)K + k] = vpo_f32_to_bf16(sq + b);
    }
  }
}

/* Dequantizing embedding gather, gpu-kernels/metal/ops/llm_elementwise.metal:1676-1701:
 * out[t, h] = T(s * q + b) of table row ids[t] -- the dequant expression above applied
 * to the selected rows.  Rows with an id outside [0, vocab) are zero-filled here
 * (the reference does not check). */
void vpo_embed_gather_w4g64_bf16(const int32_t* ids, const uint32_t* w, const uint16_t* scales,
                                 const uint16_t* biases, uint16_t* out, int H, int T, int vocab)
{
  const int Hw = H / 8, Hg = H / VPO_GROUP;
  for (size_t t = 0; t < (size_t)T; ++t) {
    const int id = ids[t];
    for (int h = 0; h < H; ++h) {
      uint16_t v = 0;
      if (id >= 0 && id < vocab) {
        const float s = vpo_bf16_to_f32(scales[(size_t)id * Hg + h / VPO_GROUP]);
        const float b = vpo_bf16_to_f32(biases[(size_t)id * Hg + h / VPO_GROUP]);
        const float sq = s * (float)nibble(w, (size_t)id, Hw, h);
        v = vpo_f32_to_bf16(sq + b);
      }
      out[t * (size_t)H + h] = v;
    }
  }
}

/* Greedy argmax of a row of logits, gpu-kernels/metal/ops/llm_elementwise.metal:2906-2941: the
 * result of its strided scans and its lowest-index tie-break is the one of a left-to-right scan
 * that takes an entry only when it is strictly greater -- the lowest index among the maxima; a
 * NaN compares false and never wins; best starts at -inf with index 0.  An entry equal to -inf is
 * taken over the initial index by the two-stage twin (:2995-3000: `val == best && i < bi`), which is
 * what is restated here, so a leading NaN is never the answer while a finite or -inf entry exists. */
void vpo_argmax_bf16(const uint16_t* logits, int32_t* out_id, int V, int rows)
{
  for (int r = 0; r < rows; ++r) {
    const uint16_t* src = logits + (size_t)r * (size_t)V;
    float best = -INFINITY;
    int bi = -1;
    for (int i = 0; i < V; ++i) {
      const float v = vpo_bf16_to_f32(src[i]);
      if (v > best || (bi < 0 && v == best)) { best = v; bi = i; }
    }
    out_id[r] = bi < 0 ? 0 : bi;
  }
}

/* ---- the stochastic sampler tail ------------------------------------------
 * gpu-kernels/metal/ops/llm_elementwise.metal:3063-3298 (`sample_topp_f16`): repetition and presence penalty ->
 * temperature -> softmax weights (cached in the element type) -> top-k, min-p, top-p as weight thresholds found by
 * bisection -> Gumbel-max draw over the kept set with a hash of (seed, index), lowest index on ties; 0 if nothing
 * is kept; the drawn token is marked seen.  The reference leaves the last bits of exp, log and of its reduction
 * order to Metal; they are pinned here to explicit fp32 operations (this file is compiled without contraction):
 *   exp, log    the Cephes single-precision polynomials, written out;
 *   reductions  thread t of 1024 takes the indices t, t + 1024, ... in ascending order, the 1024 partial results
 *               meet in a halving tree a[t] op= a[t + s], s = 512 .. 1 (the reference's own loop, :3141-3146). */
#define VPO_SAMPLE_THREADS 1024

float vpo_sample_exp(float x)
{
  if (!(x >= -87.0f)) { return 0.0f; }
  const float n = rintf(x * 1.44269504088896341f);
  float r = x - n * 0.693359375f;
  r = r - n * -2.12194440e-4f;
  float p = 1.9875691500e-4f;
  p = p * r + 1.3981999507e-3f;
  p = p * r + 8.3334519073e-3f;
  p = p * r + 4.1665795894e-2f;
  p = p * r + 1.6666665459e-1f;
  p = p * r + 5.0000001201e-1f;
  p = p * (r * r) + r;
  p = p + 1.0f;
  union { uint32_t u; float f; } sc;
  sc.u = (uint32_t)((int)n + 127) << 23;
  return p * sc.f;
}

float vpo_sample_log(float x)
{
  union { uint32_t u; float f; } v;
  v.f = x;
  int e = (int)(v.u >> 23) - 126;
  v.u = (v.u & 0x007fffffu) | 0x3f000000u;
  float m = v.f;
  if (m < 0.707106781186547524f) {
    e -= 1;
    m = m + m - 1.0f;
  } else {
    m = m - 1.0f;
  }
  const float z = m * m;
  float y = 7.0376836292e-2f;
  y = y * m + -1.1514610310e-1f;
  y = y * m + 1.1676998740e-1f;
  y = y * m + -1.2420140846e-1f;
  y = y * m + 1.4249322787e-1f;
  y = y * m + -1.6668057665e-1f;
  y = y * m + 2.0000714765e-1f;
  y = y * m + -2.4999993993e-1f;
  y = y * m + 3.3333331174e-1f;
  y = y * m * z;
  const float fe = (float)e;
  y = y + fe * -2.12194440e-4f;
  y = y - 0.5f * z;
  float r = m + y;
  r = r + fe * 0.693359375f;
  return r;
}

/* llm_elementwise.metal:3096-3104 */
float vpo_sample_hash_u01(uint32_t x)
{
  x ^= x >> 16; x *= 0x7feb352dU;
  x ^= x >> 15; x *= 0x846ca68bU;
  x ^= x >> 16;
  return ((float)x + 0.5f) * (1.0f / 4294967296.0f);
}

/* llm_elementwise.metal:3106-3113 */
static float vpo_sample_eff(float v, int seen, float rep, float pres)
{
  if (seen) {
    v = (v >= 0.0f) ? (v / rep) : (v * rep);
    v -= pres;
  }
  return v;
}

static float vpo_tree_f(float* a, int is_max)
{
  for (int s = VPO_SAMPLE_THREADS >> 1; s > 0; s >>= 1) {
    for (int t = 0; t < s; ++t) { a[t] = is_max ? (a[t] > a[t + s] ? a[t] : a[t + s]) : (a[t] + a[t + s]); }
  }
  return a[0];
}

/* ws [V] receives the cached weights (element type), seen [V] is read and the drawn token set; returns the token. */
int32_t vpo_sample_topp_bf16(const uint16_t* logits, int V, float temp, float top_p, uint32_t seed, uint16_t* ws,
                             int n_iter, float rep, float pres, int top_k, float min_p, uint8_t* seen)
{
  const int T = VPO_SAMPLE_THREADS;
  float tg[VPO_SAMPLE_THREADS];
  int tgi[VPO_SAMPLE_THREADS];
  const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
  for (int t = 0; t < T; ++t) {
    float m = -INFINITY;
    for (int i = t; i < V; i += T) {
      const float e = vpo_sample_eff(vpo_bf16_to_f32(logits[i]), seen[i] != 0, rep, pres);
      m = e > m ? e : m;
    }
    tg[t] = m;
  }
  const float maxl = vpo_tree_f(tg, 1);
  for (int t = 0; t < T; ++t) {
    float z = 0.0f;
    for (int i = t; i < V; i += T) {
      const float e = vpo_sample_eff(vpo_bf16_to_f32(logits[i]), seen[i] != 0, rep, pres);
      const float w = vpo_sample_exp((e - maxl) * inv_t);
      ws[i] = vpo_f32_to_bf16(w);
      z = z + w;
    }
    tg[t] = z;
  }
  const float Z = vpo_tree_f(tg, 0);
  const float target = top_p * Z;
  float t_k = 0.0f;
  if (top_k > 0 && top_k < V) {
    float lo = 0.0f, hi = 1.0f;
    for (int it = 0; it < n_iter; ++it) {
      const float mid = 0.5f * (lo + hi);
      long C = 0;
      for (int i = 0; i < V; ++i) { C += vpo_bf16_to_f32(ws[i]) >= mid; }      /* integer: the order is irrelevant */
      if (C >= top_k) { lo = mid; } else { hi = mid; }
    }
    t_k = lo;
  }
  const float t_mp = fmaxf(min_p, 0.0f);
  const float t_floor = fmaxf(t_k, t_mp);
  float lo = t_floor, hi = 1.0f;
  for (int it = 0; it < n_iter; ++it) {
    const float mid = 0.5f * (lo + hi);
    for (int t = 0; t < T; ++t) {
      float mass = 0.0f;
      for (int i = t; i < V; i += T) {
        const float w = vpo_bf16_to_f32(ws[i]);
        if (w >= mid) { mass = mass + w; }
      }
      tg[t] = mass;
    }
    const float M = vpo_tree_f(tg, 0);
    if (M >= target) { lo = mid; } else { hi = mid; }
  }
  const float wt = fmaxf(lo, t_floor);
  for (int t = 0; t < T; ++t) {
    float best = -INFINITY;
    int bi = -1;
    for (int i = t; i < V; i += T) {
      if (vpo_bf16_to_f32(ws[i]) >= wt) {
        const float e = vpo_sample_eff(vpo_bf16_to_f32(logits[i]), seen[i] != 0, rep, pres);
        const float u = vpo_sample_hash_u01(seed ^ ((uint32_t)i * 2654435761u + 1u));
        const float a = 0.0f - vpo_sample_log(u + 1e-20f) + 1e-20f;
        const float g = 0.0f - vpo_sample_log(a);
        const float score = e * inv_t + g;
        if (score > best) { best = score; bi = i; }
      }
    }
    tg[t] = best;
    tgi[t] = bi;
  }
  for (int s = T >> 1; s > 0; s >>= 1) {
    for (int t = 0; t < s; ++t) {
      const int take = tg[t + s] > tg[t] || (tg[t + s] == tg[t] && tgi[t + s] >= 0 && (tgi[t] < 0 || tgi[t + s] < tgi[t]));
      if (take) { tg[t] = tg[t + s]; tgi[t] = tgi[t + s]; }
    }
  }
  const int pick = tgi[0] >= 0 ? tgi[0] : 0;
  seen[pick] = 1;
  return pick;
}

/* ---- the sampler over many workgroups, thresholds from a histogram ----------
 * gpu-kernels/metal/ops/llm_elementwise.metal:3255-3640 (`sample_max_partial_f16` .. `sample_pick_combine_f16`): the
 * same pipeline as above with the vocabulary cut into n_slabs contiguous slabs (slab = ceil(V / n_slabs) indices),
 * and the top-k / top-p thresholds read off a histogram of the weights instead of bisected:
 *   bins     1024, uniform in -log(w) over [0, 40): bin(w) = clamp(int(-log(max(w, 1e-30)) / (40/1024)), 0, 1023)
 *            (:3305-3314), bin 0 the largest weights; per bin a count and a mass, the mass summed per slab in
 *            fixed point (uint32 of w * 2^16, truncated; :3293-3303, 3398-3400) and then as fp32;
 *   combine  counts, masses and Z of the slabs are added in slab order 0, 1, ... (:3432-3452);
 *   thresh   a scan from bin 0 down: t_k = low edge exp(-(b+1) * 40/1024) of the bin where the running count first
 *            reaches top_k (0 < top_k < V), t_p that of the bin where the running mass first reaches top_p * Z;
 *            wt = max(t_k, max(min_p, 0), t_p); a target never reached leaves its threshold 0 (:3461-3497);
 *   pick     Gumbel-max over {ws_i >= wt} per slab, lowest index on ties, then over the slabs (:3499-3600).
 * Fixed here as above: exp / log are the written-out polynomials; inside a slab a thread t of 256 takes the indices
 * lo + t, lo + t + 256, ... in ascending order and the 256 partial sums meet in a halving tree.  wt_out (nullable)
 * receives the threshold. */
#define VPO_HIST_THREADS 256
#define VPO_HIST_BINS 1024

static int vpo_sample_bin(float w)
{
  const float lw = 0.0f - vpo_sample_log(w > 1e-30f ? w : 1e-30f);
  int b = (int)(lw / (40.0f / 1024.0f));
  if (b < 0) { b = 0; }
  if (b >= VPO_HIST_BINS) { b = VPO_HIST_BINS - 1; }
  return b;
}

int32_t vpo_sample_hist_bf16(const uint16_t* logits, int V, float temp, float top_p, uint32_t seed, uint16_t* ws,
                             float rep, float pres, int top_k, float min_p, uint8_t* seen, int n_slabs, float* wt_out)
{
  const int T = VPO_HIST_THREADS, B = VPO_HIST_BINS;
  const int slab = (V + n_slabs - 1) / n_slabs;
  const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
  const float binw = 40.0f / 1024.0f;
  float tg[VPO_HIST_THREADS];
  int tgi[VPO_HIST_THREADS];
  /* pass A: the largest penalised logit (a maximum: no order) */
  float maxl = -INFINITY;
  for (int i = 0; i < V; ++i) {
    const float e = vpo_sample_eff(vpo_bf16_to_f32(logits[i]), seen[i] != 0, rep, pres);
    maxl = e > maxl ? e : maxl;
  }
  /* pass B: weights, per slab a partial Z and a histogram; combined in slab order */
  float* hist = (float*)calloc((size_t)(2 * B), sizeof(float));
  uint32_t* cnt = (uint32_t*)malloc((size_t)B * sizeof(uint32_t));
  uint32_t* mass = (uint32_t*)malloc((size_t)B * sizeof(uint32_t));
  float Z = 0.0f;
  for (int g = 0; g < n_slabs; ++g) {
    const int lo = g * slab;
    const int hi = lo + slab < V ? lo + slab : V;
    memset(cnt, 0, (size_t)B * sizeof(uint32_t));
    memset(mass, 0, (size_t)B * sizeof(uint32_t));
    for (int t = 0; t < T; ++t) {
      float z = 0.0f;
      for (int i = lo + t; i < hi; i += T) {
        const float e = vpo_sample_eff(vpo_bf16_to_f32(logits[i]), seen[i] != 0, rep, pres);
        const float w = vpo_sample_exp((e - maxl) * inv_t);
        ws[i] = vpo_f32_to_bf16(w);
        z = z + w;
        const int b = vpo_sample_bin(w);
        cnt[b] += 1u;
        mass[b] += (uint32_t)(w * 65536.0f);
      }
      tg[t] = z;
    }
    for (int s = T >> 1; s > 0; s >>= 1) {
      for (int t = 0; t < s; ++t) { tg[t] = tg[t] + tg[t + s]; }
    }
    Z = Z + tg[0];
    for (int b = 0; b < B; ++b) {
      hist[b] = hist[b] + (float)cnt[b];
      hist[B + b] = hist[B + b] + (float)mass[b] * (1.0f / 65536.0f);
    }
  }
  /* thresholds: the reference's single scan from bin 0 (:3476-3489), one running count and one running mass */
  const float target = top_p * Z;
  float t_k = 0.0f, t_p = 0.0f, cum_cnt = 0.0f, cum_mass = 0.0f;
  int have_k = 0, have_p = 0;
  const int do_k = top_k > 0 && top_k < V;
  for (int b = 0; b < B; ++b) {
    cum_cnt = cum_cnt + hist[b];
    cum_mass = cum_mass + hist[B + b];
    if (do_k && !have_k && cum_cnt >= (float)top_k) { t_k = vpo_sample_exp(0.0f - (float)(b + 1) * binw); have_k = 1; }
    if (!have_p && cum_mass >= target) { t_p = vpo_sample_exp(0.0f - (float)(b + 1) * binw); have_p = 1; }
    if ((!do_k || have_k) && have_p) { break; }
  }
  free(hist); free(cnt); free(mass);
  const float wt = fmaxf(fmaxf(t_k, fmaxf(min_p, 0.0f)), t_p);
  if (wt_out) { *wt_out = wt; }
  /* pass C: Gumbel-max per slab, then over the slabs */
  float best_all = -INFINITY;
  int bi_all = -1;
  for (int g = 0; g < n_slabs; ++g) {
    const int lo = g * slab;
    const int hi = lo + slab < V ? lo + slab : V;
    for (int t = 0; t < T; ++t) {
      float best = -INFINITY;
      int bi = -1;
      for (int i = lo + t; i < hi; i += T) {
        if (vpo_bf16_to_f32(ws[i]) >= wt) {
          const float e = vpo_sample_eff(vpo_bf16_to_f32(logits[i]), seen[i] != 0, rep, pres);
          const float u = vpo_sample_hash_u01(seed ^ ((uint32_t)i * 2654435761u + 1u));
          const float a = 0.0f - vpo_sample_log(u + 1e-20f) + 1e-20f;
          const float gum = 0.0f - vpo_sample_log(a);
          const float score = e * inv_t + gum;
          if (score > best) { best = score; bi = i; }
        }
      }
      tg[t] = best;
      tgi[t] = bi;
    }
    for (int s = T >> 1; s > 0; s >>= 1) {
      for (int t = 0; t < s; ++t) {
        const int take = tg[t + s] > tg[t] || (tg[t + s] == tg[t] && tgi[t + s] >= 0 && (tgi[t] < 0 || tgi[t + s] < tgi[t]));
        if (take) { tg[t] = tg[t + s]; tgi[t] = tgi[t + s]; }
      }
    }
    if (tgi[0] >= 0 && (tg[0] > best_all || (tg[0] == best_all && (bi_all < 0 || tgi[0] < bi_all)))) {
      best_all = tg[0];
      bi_all = tgi[0];
    }
  }
  const int pick = bi_all >= 0 ? bi_all : 0;
  seen[pick] = 1;
  return pick;
}

/* ---- a2/a3: QMV -------------------------------------------------------- */

/* The CPU reference loop of the reference's own QMV test,
 * tests/unit-tests/metal-lm/quant-gemv.cc:255-265:
 *     acc(double) += (double)x[k] * (s*(float)q + b)        (inner term in fp32)
 * It is the un-rounded-weight semantics of the Metal QMV kernels
 * (gpu-kernels/metal/quant/affine_qmv.metal:151-174: scale*sum(x*q) +
 * bias*sum(x), never rounding the weight to the element type).  y64 receives
 * the double sums [M,N]; y_bf16 (nullable) their RNE cast, after adding
 * residual[M,N] (nullable) the way affine_qmv_w4g64_add does
 * (affine_qmv.metal:264-266: the fp32 result is cast to the element type,
 * THEN the residual is added in the element type). */
void vpo_qmv_w4g64(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, double* y64, uint16_t* y_bf16,
                   int K, int N, int M, const uint16_t* residual)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_bf16_to_f32(scales[n * Kg + k / VPO_GROUP]);
      const float b = vpo_bf16_to_f32(biases[n * Kg + k / VPO_GROUP]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      wrow[k] = sq + b;
    }
    for (size_t m = 0; m < (size_t)M; ++m) {
      double acc = 0.0;
      const uint16_t* xr = x + m * (size_t)K;
      for (int k = 0; k < K; ++k) { acc += (double)vpo_bf16_to_f32(xr[k]) * (double)wrow[k]; }
      if (y64) { y64[m * (size_t)N + n] = acc; }
      if (y_bf16) {
        uint16_t v = vpo_f32_to_bf16((float)acc);
        if (residual) {
          v = vpo_f32_to_bf16(vpo_bf16_to_f32(v) + vpo_bf16_to_f32(residual[m * (size_t)N + n]));
        }
        y_bf16[m * (size_t)N + n] = v;
      }
    }
  }
  free(wrow);
}

/* group-32 twins of the QMV, gpu-kernels/metal/quant/affine_qmv.metal:305-342 (`affine_qmv_w4g32`,
 * `affine_qmv_w4g32_q40`) and their `_add` forms (:367-403): the loop above with a scale and a
 * bias per 32 values.  scale_only != 0 is the Q4_0 form, which never reads `biases` (may be NULL)
 * and uses b = -8 * s, exact in fp32 (affine_qmv.metal:252-256). */
void vpo_qmv_w4g32(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, double* y64, uint16_t* y_bf16,
                   int K, int N, int M, const uint16_t* residual, int scale_only)
{
  const int Kw = K / 8, Kg = K / 32;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_bf16_to_f32(scales[n * Kg + k / 32]);
      const float b = scale_only ? -8.0f * s : vpo_bf16_to_f32(biases[n * Kg + k / 32]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      wrow[k] = sq + b;
    }
    for (size_t m = 0; m < (size_t)M; ++m) {
      double acc = 0.0;
      const uint16_t* xr = x + m * (size_t)K;
      for (int k = 0; k < K; ++k) { acc += (double)vpo_bf16_to_f32(xr[k]) * (double)wrow[k]; }
      if (y64) { y64[m * (size_t)N + n] = acc; }
      if (y_bf16) {
        uint16_t v = vpo_f32_to_bf16((float)acc);
        if (residual) {
          v = vpo_f32_to_bf16(vpo_bf16_to_f32(v) + vpo_bf16_to_f32(residual[m * (size_t)N + n]));
        }
        y_bf16[m * (size_t)N + n] = v;
      }
    }
  }
  free(wrow);
}

/* The kernel's own algebra, gpu-kernels/metal/quant/affine_qmv.metal:151-174
 * (qdot) and :228-258 (block loop): per (row, group) the two sums sum(x*q) and
 * sum(x) are formed and combined as scale*accum + sum*bias.  Here both sums and
 * the running result are kept in double (the reference keeps fp32 and, for
 * bf16, forms sum(x) in bf16 quad sums -- affine_qmv.metal:60-67 -- which this
 * restatement deliberately does not copy).  Exists to show that the factored
 * form and the direct form above are the same number. */
void vpo_qmv_w4g64_factored(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            const uint16_t* x, double* y64, int K, int N, int M)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  for (size_t m = 0; m < (size_t)M; ++m) {
    const uint16_t* xr = x + m * (size_t)K;
    for (size_t n = 0; n < (size_t)N; ++n) {
      double acc = 0.0;
      for (int g = 0; g < Kg; ++g) {
        double sxq = 0.0, sx = 0.0;
        for (int k = g * VPO_GROUP; k < (g + 1) * VPO_GROUP; ++k) {
          const double xv = (double)vpo_bf16_to_f32(xr[k]);
          sxq += xv * (double)nibble(w, n, Kw, k);
          sx += xv;
        }
        acc += (double)vpo_bf16_to_f32(scales[n * Kg + g]) * sxq +
               sx * (double)vpo_bf16_to_f32(biases[n * Kg + g]);
      }
      y64[m * (size_t)N + n] = acc;
    }
  }
}

/* ---- a6/a7/a8 (+a10): QMM with optional LoRA --------------------------- */

/* t[M,r] of a runtime LoRA: gpu-kernels/metal/gemm/dense_gemm_mma.metal:227-273
 * (SCALED tile: the fp32 contraction x.A^T lands in an element-typed
 * cooperative tensor, then `(elt)((float)*it * scale)` -- two roundings) with A
 * in checkpoint orientation [r,K] (generative-models/lora-fusion.h:20-27).
 * Contraction in double. */
void vpo_lora_t(const uint16_t* x, const uint16_t* A, uint16_t* t, int M, int K, int r, float alpha)
{
  for (size_t m = 0; m < (size_t)M; ++m) {
    for (int j = 0; j < r; ++j) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) {
        acc += (double)vpo_bf16_to_f32(x[m * (size_t)K + k]) *
               (double)vpo_bf16_to_f32(A[(size_t)j * K + k]);
      }
      const float once = vpo_bf16_to_f32(vpo_f32_to_bf16((float)acc));
      t[m * (size_t)r + j] = vpo_f32_to_bf16(once * alpha);
    }
  }
}

/* Tiled quantized GEMM semantics: every QMM route of the reference rounds the
 * dequantized weight to the element type BEFORE the contraction
 * (gpu-kernels/metal/quant/affine_qmm_steel.metal:78-96 with Compute=float,
 * affine_qmm_mma.metal:96-104, affine_dequant.metal:51), accumulates in fp32
 * and rounds once on store.  With a LoRA the fused tile adds t.B^T into the
 * same accumulator before that one store
 * (gpu-kernels/metal/gemm/dense_gemm_mma.metal:297-348); B is [N,r].  The
 * contraction here is in double so the result does not depend on an order.
 * t (nullable with B) is the bf16 [M,r] produced by vpo_lora_t. */
void vpo_qmm_w4g64(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, double* y64, uint16_t* y_bf16,
                   int K, int N, int M,
                   const uint16_t* t, const uint16_t* B, int r)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_bf16_to_f32(scales[n * Kg + k / VPO_GROUP]);
      const float b = vpo_bf16_to_f32(biases[n * Kg + k / VPO_GROUP]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      wrow[k] = vpo_bf16_to_f32(vpo_f32_to_bf16(sq + b));
    }
    for (size_t m = 0; m < (size_t)M; ++m) {
      double acc = 0.0;
      const uint16_t* xr = x + m * (size_t)K;
      for (int k = 0; k < K; ++k) { acc += (double)vpo_bf16_to_f32(xr[k]) * (double)wrow[k]; }
      if (t && B) {
        for (int j = 0; j < r; ++j) {
          acc += (double)vpo_bf16_to_f32(t[m * (size_t)r + j]) *
                 (double)vpo_bf16_to_f32(B[n * (size_t)r + j]);
        }
      }
      if (y64) { y64[m * (size_t)N + n] = acc; }
      if (y_bf16) { y_bf16[m * (size_t)N + n] = vpo_f32_to_bf16((float)acc); }
    }
  }
  free(wrow);
}

/* ---- fused gate|up + SwiGLU --------------------------------------------- */

/* The load-time interleave of two row-major arrays with equal rows,
 * generative-models/llama3/metal-llama-model.cc:151-188: out row 2g = a row g
 * (gate), out row 2g+1 = b row g (up); applied alike to codes, scales, biases. */
void vpo_interleave_rows(const void* a, const void* b, void* out, size_t row_bytes, size_t rows)
{
  for (size_t g = 0; g < rows; ++g) {
    memcpy((char*)out + (2 * g) * row_bytes, (const char*)a + g * row_bytes, row_bytes);
    memcpy((char*)out + (2 * g + 1) * row_bytes, (const char*)b + g * row_bytes, row_bytes);
  }
}

/* The SwiGLU store of the fused gate|up kernels: the sums of an interleaved
 * [N = 2*ffn, K] pack arrive as y[m, 2g] = gate, y[m, 2g+1] = up and leave as
 * out[m, g] = T( (gate / (1 + exp(-gate))) * up ), evaluated on the un-rounded
 * accumulators (gpu-kernels/metal/quant/affine_qmv.metal:882-888 for the GEMV,
 * affine_qmm_steel.metal:755-766 for the GEMM; the kernels hold fp32 sums, the
 * oracle applies the same expression to its double sums).  out64 [M,N/2]
 * double; out_bf16 (nullable) its RNE cast. */
void vpo_swiglu_pairs(const double* y, double* out64, uint16_t* out_bf16, int M, int N)
{
  const int F = N / 2;
  for (size_t m = 0; m < (size_t)M; ++m) {
    for (int g = 0; g < F; ++g) {
      const double ga = y[m * (size_t)N + 2 * g], up = y[m * (size_t)N + 2 * g + 1];
      const double v = (ga / (1.0 + exp(-ga))) * up;
      if (out64) { out64[m * (size_t)F + g] = v; }
      if (out_bf16) { out_bf16[m * (size_t)F + g] = vpo_f32_to_bf16((float)v); }
    }
  }
}

/* The GEGLU twin of vpo_swiglu_pairs: out[m, g] = T(0.5 * gate * (1 + tanh(k0 * (gate +
 * 0.044715 * gate^3))) * up), k0 = sqrt(2/pi) as the reference writes it
 * (gpu-kernels/metal/quant/affine_qmv.metal:1423-1429, affine_qmm_steel.metal:1541-1544);
 * evaluated in double on the double sums. */
void vpo_geglu_pairs(const double* y, double* out64, uint16_t* out_bf16, int M, int N)
{
  const int F = N / 2;
  const double k0 = 0.7978845608028654;
  for (size_t m = 0; m < (size_t)M; ++m) {
    for (int g = 0; g < F; ++g) {
      const double ga = y[m * (size_t)N + 2 * g], up = y[m * (size_t)N + 2 * g + 1];
      const double t = tanh(k0 * (ga + 0.044715 * ga * ga * ga));
      const double v = 0.5 * ga * (1.0 + t) * up;
      if (out64) { out64[m * (size_t)F + g] = v; }
      if (out_bf16) { out_bf16[m * (size_t)F + g] = vpo_f32_to_bf16((float)v); }
    }
  }
}

/* ---- IEEE binary16 element type ----------------------------------------- */

/* The reference's kernels are templates over the element type T (VPIPE_ELT = bfloat or half,
 * apple-silicon/metal-compute/CMakeLists.txt:71-72, 159-162); these are the restatements above
 * with T = half: scales, biases, x, outputs and the residual are binary16, the arithmetic in
 * between is the same fp32 (gpu-kernels/metal/quant/affine_dequant.metal:45-52,
 * affine_qmv.metal:151-174, 264-266, affine_qmm_steel.metal:78-96). */
void vpo_dequant_w4g64_f16(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           uint16_t* out, int K, int N)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_f16_to_f32(scales[n * Kg + k / VPO_GROUP]);
      const float b = vpo_f16_to_f32(biases[n * Kg + k / VPO_GROUP]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      out[n * (size_t)K + k] = vpo_f32_to_f16(sq + b);
    }
  }
}

/* The half build of affine_dequant_w8g64 / _w8g32 (affine_dequant.metal:60-131 with VPIPE_ELT = half): one byte per
 * value, binary16 scales and biases, out = f16(fp32(s * q + b)); the product is exact (11 x 8 bit significands). */
void vpo_dequant_w8_f16(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                        uint16_t* out, int K, int N, int group)
{
  const int Kw = K / 4, Kg = K / group;
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_f16_to_f32(scales[n * Kg + k / group]);
      const float b = vpo_f16_to_f32(biases[n * Kg + k / group]);
      const uint32_t q = (w[n * Kw + k / 4] >> (8 * (k & 3))) & 0xffu;
      const float sq = s * (float)q;
      out[n * (size_t)K + k] = vpo_f32_to_f16(sq + b);
    }
  }
}

/* rounded != 0: the GEMM's weights, rounded to binary16 before the contraction; 0: the GEMV's. */
void vpo_matmul_w4g64_f16(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                          const uint16_t* x, double* y64, uint16_t* y_f16,
                          int K, int N, int M, const uint16_t* residual, int rounded)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_f16_to_f32(scales[n * Kg + k / VPO_GROUP]);
      const float b = vpo_f16_to_f32(biases[n * Kg + k / VPO_GROUP]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      wrow[k] = rounded ? vpo_f16_to_f32(vpo_f32_to_f16(sq + b)) : sq + b;
    }
    for (size_t m = 0; m < (size_t)M; ++m) {
      double acc = 0.0;
      const uint16_t* xr = x + m * (size_t)K;
      for (int k = 0; k < K; ++k) { acc += (double)vpo_f16_to_f32(xr[k]) * (double)wrow[k]; }
      if (y64) { y64[m * (size_t)N + n] = acc; }
      if (y_f16) {
        uint16_t v = vpo_f32_to_f16((float)acc);
        if (residual) {
          v = vpo_f32_to_f16(vpo_f16_to_f32(v) + vpo_f16_to_f32(residual[m * (size_t)N + n]));
        }
        y_f16[m * (size_t)N + n] = v;
      }
    }
  }
  free(wrow);
}

/* RMSNorm ahead of the fused-QKV GEMV, gpu-kernels/metal/quant/affine_qmv.metal:601-616: the sum of squares, the
 * mean and the reciprocal root in double here (the kernel: fp32), then the reference's product order in fp32,
 * T(float(x[k]) * inv * float(norm_w[k])), one rounding. */
void vpo_rmsnorm_bf16(const uint16_t* x, const uint16_t* norm_w, uint16_t* out, int K, int M, float eps)
{
  for (size_t m = 0; m < (size_t)M; ++m) {
    double sq = 0.0;
    for (int k = 0; k < K; ++k) {
      const double v = (double)vpo_bf16_to_f32(x[m * (size_t)K + k]);
      sq += v * v;
    }
    const float inv = (float)(1.0 / sqrt(sq / (double)K + (double)eps));
    for (int k = 0; k < K; ++k) {
      const float v = vpo_bf16_to_f32(x[m * (size_t)K + k]) * inv;
      out[m * (size_t)K + k] = vpo_f32_to_bf16(v * vpo_bf16_to_f32(norm_w[k]));
    }
  }
}

/* The adapter on binary16 elements: gpu-kernels/metal/gemm/dense_gemm_mma.metal:227-273 with VPIPE_ELT = half
 * (:28-33) -- t[M,r] = f16((float)f16(x . A^T) * alpha), two roundings, the contraction in double. */
void vpo_lora_t_f16(const uint16_t* x, const uint16_t* A, uint16_t* t, int M, int K, int r, float alpha)
{
  for (size_t m = 0; m < (size_t)M; ++m) {
    for (int j = 0; j < r; ++j) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) {
        acc += (double)vpo_f16_to_f32(x[m * (size_t)K + k]) * (double)vpo_f16_to_f32(A[(size_t)j * K + k]);
      }
      const float once = vpo_f16_to_f32(vpo_f32_to_f16((float)acc));
      t[m * (size_t)r + j] = vpo_f32_to_f16(once * alpha);
    }
  }
}

/* The fused GEMM on binary16 elements with the adapter's second factor in the same accumulator before the one
 * store (dense_gemm_mma.metal:297-348): y = f16(x . f16(s q + b)^T + t . B^T), B [N,r], t from vpo_lora_t_f16;
 * contraction in double. */
void vpo_qmm_lora_w4g64_f16(const uint32_t* w, const uint16_t* scales, const uint16_t* biases, const uint16_t* x,
                            double* y64, uint16_t* y_f16, int K, int N, int M, const uint16_t* t, const uint16_t* B,
                            int r)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_f16_to_f32(scales[n * Kg + k / VPO_GROUP]);
      const float b = vpo_f16_to_f32(biases[n * Kg + k / VPO_GROUP]);
      const float sq = s * (float)nibble(w, n, Kw, k);
      wrow[k] = vpo_f16_to_f32(vpo_f32_to_f16(sq + b));
    }
    for (size_t m = 0; m < (size_t)M; ++m) {
      double acc = 0.0;
      const uint16_t* xr = x + m * (size_t)K;
      for (int k = 0; k < K; ++k) { acc += (double)vpo_f16_to_f32(xr[k]) * (double)wrow[k]; }
      for (int j = 0; j < r; ++j) {
        acc += (double)vpo_f16_to_f32(t[m * (size_t)r + j]) * (double)vpo_f16_to_f32(B[n * (size_t)r + j]);
      }
      if (y64) { y64[m * (size_t)N + n] = acc; }
      if (y_f16) { y_f16[m * (size_t)N + n] = vpo_f32_to_f16((float)acc); }
    }
  }
  free(wrow);
}

/* ---- MoE prefill: the expert sort and the grouped GEMMs ------------------- */

/* gpu-kernels/metal/ops/llm_elementwise.metal:255-326 (moe_ifill_i32, moe_hist_i32,
 * moe_sort_setup_i32, moe_scatter_i32): a histogram of the pairs over the experts, every
 * expert's share rounded up to whole blocks of block_rows slots, experts ascending;
 * tile2e[t] the expert of block t (-1 unused), srow[slot] = pair / top_k, sdst[slot] = pair
 * (-1 for padding slots).  The reference hands the slots of an expert out by an atomic
 * counter (any order); this restatement takes the pairs in ascending order.  A pair with an
 * id outside [0, E) is skipped (the reference would index out of bounds).  Returns the blocks
 * in use. */
int vpo_moe_sort_pairs(const int32_t* eid, int np, int top_k, int E, int block_rows, int max_tiles,
                       int32_t* tile2e, int32_t* srow, int32_t* sdst)
{
  const int npad = max_tiles * block_rows;
  int* hist = (int*)calloc((size_t)E, sizeof(int));
  int* boff = (int*)calloc((size_t)E, sizeof(int));
  int* cursor = (int*)calloc((size_t)E, sizeof(int));
  for (int i = 0; i < npad; ++i) { srow[i] = -1; sdst[i] = -1; }
  for (int t = 0; t < max_tiles; ++t) { tile2e[t] = -1; }
  for (int p = 0; p < np; ++p) {
    if (eid[p] >= 0 && eid[p] < E) { hist[eid[p]] += 1; }
  }
  int off = 0;
  for (int e = 0; e < E; ++e) {
    boff[e] = off;
    const int nt = (hist[e] + block_rows - 1) / block_rows;
    const int t0 = off / block_rows;
    for (int t = 0; t < nt; ++t) {
      if (t0 + t < max_tiles) { tile2e[t0 + t] = e; }
    }
    off += nt * block_rows;
  }
  for (int p = 0; p < np; ++p) {
    const int e = eid[p];
    if (e < 0 || e >= E) { continue; }
    const int slot = boff[e] + cursor[e]++;
    if (slot < npad) { srow[slot] = p / top_k; sdst[slot] = p; }
  }
  free(hist); free(boff); free(cursor);
  return off / block_rows;
}

/* The grouped expert GEMMs over the sorted slots
 * (gpu-kernels/metal/quant/affine_qmm_steel.metal:1092-1170 gate|up with the gathering
 * loader :972-1020, :1367-1458 down with the scattering store): block t = slots
 * [t*block_rows, ...) multiplies the slab of expert tile2e[t] of the batched pack
 * [E, N, K/8] (a block with tile2e < 0 is skipped, its outputs untouched).
 *   srow != NULL (gate|up): x row of slot i is x[srow[i]], zeros for srow[i] < 0; the sums
 *     go to y64[i, :] (the caller applies the gated store);
 *   sdst != NULL (down): x row of slot i is x[i]; the sums go to y64[sdst[i], :] and their
 *     bf16 rounding to y_bf16[sdst[i], :] (slots with sdst < 0 write nothing).
 * Arithmetic of vpo_qmm_w4g64: bf16-rounded weights, contraction in double. */
static void qmm_grouped_bits(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            const uint16_t* x, double* y64, uint16_t* y_bf16, int K, int N, int npad,
                            int block_rows, const int32_t* tile2e, const int32_t* srow,
                            const int32_t* sdst, int bits)
{
  const int Kw = bits == 4 ? K / 8 : K / 4, Kg = K / VPO_GROUP;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
  for (int t = 0; t < npad / block_rows; ++t) {
    const int e = tile2e[t];
    if (e < 0) { continue; }
    const uint32_t* we = w + (size_t)e * N * Kw;
    const uint16_t* se = scales + (size_t)e * N * Kg;
    const uint16_t* be = biases + (size_t)e * N * Kg;
    for (size_t n = 0; n < (size_t)N; ++n) {
      for (int k = 0; k < K; ++k) {
        const float s = vpo_bf16_to_f32(se[n * Kg + k / VPO_GROUP]);
        const float b = vpo_bf16_to_f32(be[n * Kg + k / VPO_GROUP]);
        const float sq = s * (float)(bits == 4 ? nibble(we, n, Kw, k) : code8(we, n, Kw, k));
        wrow[k] = vpo_bf16_to_f32(vpo_f32_to_bf16(sq + b));
      }
      for (int i = t * block_rows; i < (t + 1) * block_rows; ++i) {
        double acc = 0.0;
        long dst = i;
        if (srow) {
          if (srow[i] >= 0) {
            const uint16_t* xr = x + (size_t)srow[i] * K;
            for (int k = 0; k < K; ++k) { acc += (double)vpo_bf16_to_f32(xr[k]) * (double)wrow[k]; }
          }
        } else {
          if (sdst[i] < 0) { continue; }
          dst = sdst[i];
          const uint16_t* xr = x + (size_t)i * K;
          for (int k = 0; k < K; ++k) { acc += (double)vpo_bf16_to_f32(xr[k]) * (double)wrow[k]; }
        }
        if (y64) { y64[(size_t)dst * N + n] = acc; }
        if (y_bf16) { y_bf16[(size_t)dst * N + n] = vpo_f32_to_bf16((float)acc); }
      }
    }
  }
  free(wrow);
}

void vpo_qmm_grouped_w4g64(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           const uint16_t* x, double* y64, uint16_t* y_bf16, int K, int N, int npad,
                           int block_rows, const int32_t* tile2e, const int32_t* srow,
                           const int32_t* sdst)
{
  qmm_grouped_bits(w, scales, biases, x, y64, y_bf16, K, N, npad, block_rows, tile2e, srow, sdst, 4);
}

/* 8-bit twins (affine_qmm_grouped_w8g64, affine_qmm_grouped_swiglu_w8g64, affine_qmm_grouped_geglu_w8g64,
 * gpu-kernels/metal/quant/affine_qmm_steel.metal:1069-1090, 1290-1312, 1341-1366: "fully bit-parameterized"):
 * one byte per value, the batched pack [E, N, K/4]. */
void vpo_qmm_grouped_w8g64(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           const uint16_t* x, double* y64, uint16_t* y_bf16, int K, int N, int npad,
                           int block_rows, const int32_t* tile2e, const int32_t* srow,
                           const int32_t* sdst)
{
  qmm_grouped_bits(w, scales, biases, x, y64, y_bf16, K, N, npad, block_rows, tile2e, srow, sdst, 8);
}

/* ---- a12: the packer --------------------------------------------------- */

/* gpu-kernels/metal/quant/affine_dequant.metal:243-285 (affine_quant_impl<4,64>):
 * per group mn/mx, optional clip toward the midpoint, scale=(mx-mn)/15,
 * inv = scale>0 ? 1/scale : 0, q = clamp(round((v-mn)*inv), 0, 15) with Metal's
 * round() = half away from zero (C roundf), scale and mn emitted as F16.
 * Host twin: generative-models/quantize/model-quantizer.cc:240-264 (lround).
 * Input is fp32 here (the kernel widens its f16/bf16 input to float first). */
/* Every width and group (affine_quant_impl<BITS, GROUP>, :243-301: bits 4 or 8, group 64 or 32). */
void vpo_quantize(const float* wsrc, uint32_t* codes, uint16_t* scales_f16, uint16_t* biases_f16, int K, int N,
                  float clip, int bits, int group)
{
  const int vpw = 32 / bits, wpg = group / vpw, qmax = (1 << bits) - 1;
  const int Kw = K / vpw, Kg = K / group;
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int g = 0; g < Kg; ++g) {
      const float* xp = wsrc + n * (size_t)K + (size_t)g * group;
      float mn = INFINITY, mx = -INFINITY;
      for (int i = 0; i < group; ++i) {
        mn = fminf(mn, xp[i]);
        mx = fmaxf(mx, xp[i]);
      }
      if (clip < 1.0f) {
        const float mid = 0.5f * (mn + mx);
        mn = mid + (mn - mid) * clip;
        mx = mid + (mx - mid) * clip;
      }
      const float scale = (mx - mn) / (float)qmax;
      const float inv = (scale > 0.0f) ? 1.0f / scale : 0.0f;
      scales_f16[n * Kg + g] = vpo_f32_to_f16(scale);
      biases_f16[n * Kg + g] = vpo_f32_to_f16(mn);
      for (int wi = 0; wi < wpg; ++wi) {
        uint32_t packed = 0;
        for (int i = 0; i < vpw; ++i) {
          int q = (int)roundf((xp[wi * vpw + i] - mn) * inv);
          q = q < 0 ? 0 : (q > qmax ? qmax : q);
          packed |= (uint32_t)q << (bits * i);
        }
        codes[n * (size_t)Kw + (size_t)g * wpg + wi] = packed;
      }
    }
  }
}

void vpo_quantize_w4g64(const float* wsrc, uint32_t* codes, uint16_t* scales_f16,
                        uint16_t* biases_f16, int K, int N, float clip)
{
  vpo_quantize(wsrc, codes, scales_f16, biases_f16, K, N, clip, 4, VPO_GROUP);
}

/* Output byte sizes, generative-models/quantize/affine-quantizer.h:37-40. */
size_t vpo_weight_bytes(int N, int K) { return (size_t)N * (size_t)(K * 4 / 32) * 4; }
size_t vpo_scale_bytes(int N, int K) { return (size_t)N * (size_t)(K / VPO_GROUP) * 2; }

/* ---- 8-bit twin (w8g64) ------------------------------------------------- */

/* 8-bit affine weights hold one byte per value, four per u32 word, little-endian
 * within the word: q[n, 4j+i] = (w[n,j] >> 8i) & 0xFF, a row is K/4 words
 * (gpu-kernels/metal/quant/affine_dequant.metal:60-97, affine_qmv.metal:68-76,
 * 168-172: qmv reads the row as raw bytes).  Scales and biases as for 4 bits,
 * one pair per 64 values. */
static inline unsigned code8(const uint32_t* w, size_t n, int Kw, int k)
{
  return (w[n * (size_t)Kw + (size_t)(k >> 2)] >> (8 * (k & 3))) & 0xffu;
}

/* affine_dequant_w8g64 (affine_dequant.metal:68-97): out = (elt)(s * (float)q + b);
 * s*q is exact in fp32 (8-bit x 8-bit significands). */
void vpo_dequant_w8_bf16(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                         uint16_t* out, int K, int N, int group)
{
  const int Kw = K / 4, Kg = K / group;
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_bf16_to_f32(scales[n * Kg + k / group]);
      const float b = vpo_bf16_to_f32(biases[n * Kg + k / group]);
      const float sq = s * (float)code8(w, n, Kw, k);
      out[n * (size_t)K + k] = vpo_f32_to_bf16(sq + b);
    }
  }
}

/* affine_requant_w8_to_w4_g64 (affine_dequant.metal:134-186): per group of 64, expand the 8-bit codes to fp32
 * (v = s8 * q8 + b8, the product exact), take min and max, and quantize again to 4 bits with
 * scale = (max - min) / 15, bias = min, q4 = round((v - min) * (1 / scale)) (halves away from zero, as Metal's
 * round) clamped to 0..15; a constant group gives scale 0 and all codes 0.  The stored scale and bias are the
 * element-type roundings; the codes are computed with the unrounded fp32 scale.  Divisions are IEEE here (Metal's
 * default fast division may differ in the last bit: only an Apple-GPU run could pin that bit). */
void vpo_requant_w8_to_w4_g64(const uint32_t* w8, const uint16_t* s8, const uint16_t* b8,
                              uint32_t* w4, uint16_t* s4, uint16_t* b4, int K, int N)
{
  const int Kw8 = K / 4, Kw4 = K / 8, Kg = K / VPO_GROUP;
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int g = 0; g < Kg; ++g) {
      const float s = vpo_bf16_to_f32(s8[n * Kg + g]);
      const float b = vpo_bf16_to_f32(b8[n * Kg + g]);
      float v[VPO_GROUP];
      float mn = INFINITY, mx = -INFINITY;
      for (int i = 0; i < VPO_GROUP; ++i) {
        const float sq = s * (float)code8(w8, n, Kw8, g * VPO_GROUP + i);
        v[i] = sq + b;
        mn = v[i] < mn ? v[i] : mn;
        mx = v[i] > mx ? v[i] : mx;
      }
      const float scale = (mx - mn) / 15.0f;
      const float inv = scale > 0.0f ? 1.0f / scale : 0.0f;
      s4[n * Kg + g] = vpo_f32_to_bf16(scale);
      b4[n * Kg + g] = vpo_f32_to_bf16(mn);
      for (int wi = 0; wi < VPO_GROUP / 8; ++wi) {
        uint32_t packed = 0;
        for (int i = 0; i < 8; ++i) {
          const float d = v[wi * 8 + i] - mn;
          int q = (int)roundf(d * inv);
          q = q < 0 ? 0 : (q > 15 ? 15 : q);
          packed |= (uint32_t)q << (4 * i);
        }
        w4[n * Kw4 + (size_t)g * (VPO_GROUP / 8) + wi] = packed;
      }
    }
  }
}

void vpo_dequant_w8g64_bf16(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            uint16_t* out, int K, int N)
{
  vpo_dequant_w8_bf16(w, scales, biases, out, K, N, VPO_GROUP);
}

/* QMV (affine_qmv_w8g64, affine_qmv.metal:3034-3050 = qmv_fast_impl<T,64,8>: the same
 * factored sum scale*sum(x*q) + bias*sum(x), weight never rounded) when rounded == 0;
 * the GEMM semantics (weight rounded to the element type first: affine_qmm_steel_w8g64,
 * affine_qmm_steel.metal:1601-1624, and the dequant-once route) when rounded != 0.
 * Double accumulation; y_bf16 (nullable) is the RNE cast. */
/* The group is a parameter: 64, or 32 for the twins of affine_dequant.metal:99-131, affine_qmv.metal:3053-3069,
 * affine_qmm_steel.metal:1674-1698, in which only the stride of the scales changes. */
void vpo_matmul_w8(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, double* y64, uint16_t* y_bf16, int K, int N, int M, int rounded, int group);
void vpo_matmul_w8g64(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                      const uint16_t* x, double* y64, uint16_t* y_bf16, int K, int N, int M, int rounded)
{
  vpo_matmul_w8(w, scales, biases, x, y64, y_bf16, K, N, M, rounded, VPO_GROUP);
}

void vpo_matmul_w8(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, double* y64, uint16_t* y_bf16, int K, int N, int M, int rounded, int group)
{
  const int Kw = K / 4, Kg = K / group;
  float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
  for (size_t n = 0; n < (size_t)N; ++n) {
    for (int k = 0; k < K; ++k) {
      const float s = vpo_bf16_to_f32(scales[n * Kg + k / group]);
      const float b = vpo_bf16_to_f32(biases[n * Kg + k / group]);
      const float sq = s * (float)code8(w, n, Kw, k);
      const float v = sq + b;
      wrow[k] = rounded ? vpo_bf16_to_f32(vpo_f32_to_bf16(v)) : v;
    }
    for (size_t m = 0; m < (size_t)M; ++m) {
      double acc = 0.0;
      const uint16_t* xr = x + m * (size_t)K;
      for (int k = 0; k < K; ++k) { acc += (double)vpo_bf16_to_f32(xr[k]) * (double)wrow[k]; }
      if (y64) { y64[m * (size_t)N + n] = acc; }
      if (y_bf16) { y_bf16[m * (size_t)N + n] = vpo_f32_to_bf16((float)acc); }
    }
  }
  free(wrow);
}

/* ---- timed CPU baseline ------------------------------------------------ */

/* "quantize-module dequant + fp32 matmul": expand the pack to fp32 [N,K]
 * (semantics of affine_dequant.metal:25-58 / model-quantizer.cc:257) and run a
 * plain fp32 dot per output (the float-accumulating oracle loop of
 * tests/unit-tests/metal-compute-gemm-mma.cc:337-347), bf16 store.  OpenMP over
 * output rows when built with -fopenmp.  wdeq is caller-provided scratch
 * [N,K] fp32.  Returns nothing; the benchmark times the call. */
void vpo_cpu_dequant_matmul(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            const uint16_t* x, uint16_t* y, float* wdeq, float* xf,
                            int K, int N, int M)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  for (size_t i = 0; i < (size_t)M * (size_t)K; ++i) { xf[i] = vpo_bf16_to_f32(x[i]); }
#pragma omp parallel for schedule(static)
  for (long n = 0; n < (long)N; ++n) {
    float* o = wdeq + (size_t)n * K;
    for (int j = 0; j < Kw; ++j) {
      const uint32_t p = w[(size_t)n * Kw + j];
      const float s = vpo_bf16_to_f32(scales[(size_t)n * Kg + j / 8]);
      const float b = vpo_bf16_to_f32(biases[(size_t)n * Kg + j / 8]);
      for (int i = 0; i < 8; ++i) {
        const float sq = s * (float)((p >> (4 * i)) & 0xfu);
        o[j * 8 + i] = sq + b;
      }
    }
  }
#pragma omp parallel for schedule(static)
  for (long n = 0; n < (long)N; ++n) {
    const float* wr = wdeq + (size_t)n * K;
    for (size_t m = 0; m < (size_t)M; ++m) {
      const float* xr = xf + m * (size_t)K;
      float acc = 0.0f;
#pragma omp simd reduction(+ : acc)
      for (int k = 0; k < K; ++k) { acc += xr[k] * wr[k]; }
      y[m * (size_t)N + (size_t)n] = vpo_f32_to_bf16(acc);
    }
  }
}

/* The two stages of the baseline on their own, and the fused form (each weight expanded in a register
 * and multiplied at once, no fp32 matrix in memory): same expressions, same order of the sum. */
void vpo_cpu_dequant_f32(const uint32_t* w, const uint16_t* scales, const uint16_t* biases, float* wdeq,
                         int K, int N)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
#pragma omp parallel for schedule(static)
  for (long n = 0; n < (long)N; ++n) {
    float* o = wdeq + (size_t)n * K;
    for (int j = 0; j < Kw; ++j) {
      const uint32_t p = w[(size_t)n * Kw + j];
      const float s = vpo_bf16_to_f32(scales[(size_t)n * Kg + j / 8]);
      const float b = vpo_bf16_to_f32(biases[(size_t)n * Kg + j / 8]);
      for (int i = 0; i < 8; ++i) {
        const float sq = s * (float)((p >> (4 * i)) & 0xfu);
        o[j * 8 + i] = sq + b;
      }
    }
  }
}

void vpo_cpu_matmul_f32(const float* wdeq, const uint16_t* x, uint16_t* y, float* xf, int K, int N, int M)
{
  for (size_t i = 0; i < (size_t)M * (size_t)K; ++i) { xf[i] = vpo_bf16_to_f32(x[i]); }
#pragma omp parallel for schedule(static)
  for (long n = 0; n < (long)N; ++n) {
    const float* wr = wdeq + (size_t)n * K;
    for (size_t m = 0; m < (size_t)M; ++m) {
      const float* xr = xf + m * (size_t)K;
      float acc = 0.0f;
#pragma omp simd reduction(+ : acc)
      for (int k = 0; k < K; ++k) { acc += xr[k] * wr[k]; }
      y[m * (size_t)N + (size_t)n] = vpo_f32_to_bf16(acc);
    }
  }
}

void vpo_cpu_fused_qmv(const uint32_t* w, const uint16_t* scales, const uint16_t* biases, const uint16_t* x,
                       uint16_t* y, float* xf, int K, int N, int M)
{
  const int Kw = K / 8, Kg = K / VPO_GROUP;
  for (size_t i = 0; i < (size_t)M * (size_t)K; ++i) { xf[i] = vpo_bf16_to_f32(x[i]); }
#pragma omp parallel for schedule(static)
  for (long n = 0; n < (long)N; ++n) {
    for (size_t m = 0; m < (size_t)M; ++m) {
      const float* xr = xf + m * (size_t)K;
      float acc = 0.0f;
      for (int j = 0; j < Kw; ++j) {
        const uint32_t p = w[(size_t)n * Kw + j];
        const float s = vpo_bf16_to_f32(scales[(size_t)n * Kg + j / 8]);
        const float b = vpo_bf16_to_f32(biases[(size_t)n * Kg + j / 8]);
        for (int i = 0; i < 8; ++i) {
          const float sq = s * (float)((p >> (4 * i)) & 0xfu);
          acc += xr[j * 8 + i] * (sq + b);
        }
      }
      y[m * (size_t)N + (size_t)n] = vpo_f32_to_bf16(acc);
    }
  }
}

#ifdef _OPENMP
#include <omp.h>
int vpo_num_threads(void) { return omp_get_max_threads(); }
#else
int vpo_num_threads(void) { return 1; }
#endif

// Stochastic tail of a decode step: the full sampler over one row of logits, on the device, so that the
// drawn token never leaves it (gpu-kernels/metal/ops/llm_elementwise.metal:3063-3298, `sample_topp_f16`).
// One workgroup.  The pipeline and its order are the reference's:
//   repetition penalty -> presence penalty -> temperature -> softmax weights -> top-k -> min-p -> top-p
//   -> multinomial draw by the Gumbel-max trick,
// with the three filters as weight thresholds (no sort of the vocabulary):
//   eff_i  = seen[i] ? (v >= 0 ? v / rep : v * rep) - pres : v                         (:3106-3113)
//   w_i    = exp((eff_i - max eff) / temp), cached in `ws` in the element type; Z = sum of the w_i (fp32, unrounded)
//   t_k    = largest t of a bisection of [0, 1] with count{ws_i >= t} >= top_k           (:3170-3193; 0 < top_k < V)
//   floor  = max(t_k, min_p)   (the largest weight is 1, so min-p's probability floor is a weight floor)
//   wt     = largest t of a bisection of [floor, 1] with sum{ws_i : ws_i >= t} >= top_p Z (:3203-3222)
//   pick   = argmax over {ws_i >= wt} of eff_i / temp - log(-log(u_i)), u_i a hash of (seed, i), lowest index on
//            ties; 0 if nothing is kept; seen[pick] = 1                                   (:3224-3262)
//
// What is fixed here beyond the reference (Metal's fast math and reduction order are not defined to the bit): every
// floating-point step is written so that a plain C restatement gives the same bits -- exp and log are polynomials
// over explicit fp32 multiplies and adds (no contraction into fma in this file), a thread takes the indices
// t, t + 1024, ... in ascending order and the 1024 partial results meet in a halving tree
// (a[t] op= a[t + s], s = 512 .. 1), the reference's own pattern.  The draw is therefore an exact function of
// (logits, seen, parameters, seed), checked as index work, not to a tolerance.
#include "vpq_device.h"
#include "vpq_internal.h"

#pragma clang fp contract(off)

namespace vpq {

namespace {

constexpr int kSampleThreads = 1024;

// exp(x) for x <= 0: 2^n * p(r), n = rint(x log2 e), r = x - n ln 2 in two pieces, p the degree-5 polynomial of
// the Cephes expf.  Below -87 the result is 0.
__device__ __forceinline__ float sample_exp(float x)
{
  if (!(x >= -87.0f)) { return 0.0f; }
  const float n = __builtin_rintf(x * 1.44269504088896341f);
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
  return p * __uint_as_float((uint32_t)((int)n + 127) << 23);
}

// log(x) for normal x > 0 (the Cephes logf): x = m 2^e with m in [sqrt(1/2), sqrt(2)), a degree-8 polynomial in
// m - 1, e ln 2 added in two pieces.
__device__ __forceinline__ float sample_log(float x)
{
  const uint32_t bits = __float_as_uint(x);
  int e = (int)(bits >> 23) - 126;
  float m = __uint_as_float((bits & 0x007fffffu) | 0x3f000000u);      // [0.5, 1)
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

// (llm_elementwise.metal:3096-3104) bias-reduced integer hash -> uniform in (0, 1]
__device__ __forceinline__ float sample_hash_u01(uint32_t x)
{
  x ^= x >> 16; x *= 0x7feb352dU;
  x ^= x >> 15; x *= 0x846ca68bU;
  x ^= x >> 16;
  return ((float)x + 0.5f) * (1.0f / 4294967296.0f);
}

__device__ __forceinline__ float sample_eff(float v, bool seen, float rep, float pres)
{
  if (seen) {
    v = (v >= 0.0f) ? (v / rep) : (v * rep);
    v -= pres;
  }
  return v;
}

template <typename T, typename Op>
__device__ __forceinline__ T tree(T* a, T mine, Op op)
{
  const int t = threadIdx.x;
  a[t] = mine;
  __syncthreads();
  for (int s = kSampleThreads >> 1; s > 0; s >>= 1) {
    if (t < s) { a[t] = op(a[t], a[t + s]); }
    __syncthreads();
  }
  const T r = a[0];
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(kSampleThreads) void sample_topp_kernel(
    const uint16_t* __restrict__ logits, int32_t* __restrict__ out_id, int V, float temp, float top_p, uint32_t seed,
    uint16_t* __restrict__ ws, int n_iter, float rep, float pres, int top_k, float min_p, uint8_t* __restrict__ seen)
{
  __shared__ float tg[kSampleThreads];
  __shared__ int tgi[kSampleThreads];
  const int t = threadIdx.x;
  const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
  auto fmax_op = [](float a, float b) { return a > b ? a : b; };     // a NaN on the right is never taken
  auto fadd_op = [](float a, float b) { return a + b; };
  auto iadd_op = [](int a, int b) { return a + b; };

  // 1) the largest penalised logit
  float m = -INFINITY;
  for (int i = t; i < V; i += kSampleThreads) {
    const float e = sample_eff(bf16_bits_to_f32(logits[i]), seen[i] != 0, rep, pres);
    m = e > m ? e : m;
  }
  const float maxl = tree(tg, m, fmax_op);

  // 2) the weights, cached in the element type, and their sum
  float z = 0.0f;
  for (int i = t; i < V; i += kSampleThreads) {
    const float e = sample_eff(bf16_bits_to_f32(logits[i]), seen[i] != 0, rep, pres);
    const float w = sample_exp((e - maxl) * inv_t);
    ws[i] = (uint16_t)f32_to_bf16_bits(w);
    z = z + w;
  }
  __threadfence_block();
  const float Z = tree(tg, z, fadd_op);
  const float target = top_p * Z;

  // 3a) top-k as a weight threshold
  float t_k = 0.0f;
  if (top_k > 0 && top_k < V) {
    float lo = 0.0f, hi = 1.0f;
    for (int it = 0; it < n_iter; ++it) {
      const float mid = 0.5f * (lo + hi);
      int cnt = 0;
      for (int i = t; i < V; i += kSampleThreads) {
        if (bf16_bits_to_f32(ws[i]) >= mid) { ++cnt; }
      }
      const int C = tree(tgi, cnt, iadd_op);
      if (C >= top_k) { lo = mid; } else { hi = mid; }
    }
    t_k = lo;
  }
  // 3b) min-p as a weight floor
  const float t_mp = fmaxf(min_p, 0.0f);
  const float t_floor = fmaxf(t_k, t_mp);

  // 3c) the nucleus threshold over the survivors
  float lo = t_floor, hi = 1.0f;
  for (int it = 0; it < n_iter; ++it) {
    const float mid = 0.5f * (lo + hi);
    float mass = 0.0f;
    for (int i = t; i < V; i += kSampleThreads) {
      const float w = bf16_bits_to_f32(ws[i]);
      if (w >= mid) { mass = mass + w; }
    }
    const float M = tree(tg, mass, fadd_op);
    if (M >= target) { lo = mid; } else { hi = mid; }
  }
  const float wt = fmaxf(lo, t_floor);

  // 4) Gumbel-max over the kept set, lowest index on ties
  float best = -INFINITY;
  int bi = -1;
  for (int i = t; i < V; i += kSampleThreads) {
    if (bf16_bits_to_f32(ws[i]) >= wt) {
      const float e = sample_eff(bf16_bits_to_f32(logits[i]), seen[i] != 0, rep, pres);
      const float u = sample_hash_u01(seed ^ ((uint32_t)i * 2654435761u + 1u));
      const float a = 0.0f - sample_log(u + 1e-20f) + 1e-20f;
      const float g = 0.0f - sample_log(a);
      const float score = e * inv_t + g;
      if (score > best) { best = score; bi = i; }
    }
  }
  tg[t] = best;
  tgi[t] = bi;
  __syncthreads();
  for (int s = kSampleThreads >> 1; s > 0; s >>= 1) {
    if (t < s) {
      const bool take = tg[t + s] > tg[t] || (tg[t + s] == tg[t] && tgi[t + s] >= 0 && (tgi[t] < 0 || tgi[t + s] < tgi[t]));
      if (take) { tg[t] = tg[t + s]; tgi[t] = tgi[t + s]; }
    }
    __syncthreads();
  }
  if (t == 0) {
    const int pick = tgi[0] >= 0 ? tgi[0] : 0;
    out_id[0] = pick;
    seen[pick] = 1;
  }
}

// ---- the sampler over many workgroups, thresholds from a histogram ----------------------------------------------
// (llm_elementwise.metal:3255-3640: `sample_max_partial_f16`, `sample_max_combine_f16`, `sample_zhist_partial_f16`,
// `sample_zhist_combine_f16`, `sample_thresh_f16`, `sample_pick_partial_f16`, `sample_pick_combine_f16`.)  The
// vocabulary is cut into n_slabs contiguous slabs, one workgroup of 256 threads each; top-k and top-p become the low
// edge of a histogram bin (1024 bins uniform in -log w over [0, 40), bin 0 the largest weights), so the kept set is
// the exact sampler's plus at most one bin's worth of weights.  Five launches instead of the reference's seven: the
// combine of the maxima is the prologue of the weight pass (every workgroup reduces the n_slabs maxima itself), and
// the combine of the histograms and the threshold scan are one workgroup.
//   work (fp32 words): [0, S) slab maxima | S x (2 B + 1): per slab counts, masses, Z | 2 B + 1: their sums |
//   1: the weight threshold | 2 S: per slab (best score, its index)
// Exactness as above: a thread takes lo + t, lo + t + 256, ... in ascending order, partial sums meet in a halving
// tree, slabs are added in slab order; counts and the fixed-point masses of a slab are integer sums.
constexpr int kHistThreads = 256;
constexpr int kHistBins = 1024;
constexpr float kHistBinWidth = 40.0f / 1024.0f;

__device__ __forceinline__ int sample_bin(float w)
{
  const float lw = 0.0f - sample_log(w > 1e-30f ? w : 1e-30f);
  int b = (int)(lw / kHistBinWidth);
  if (b < 0) { b = 0; }
  if (b >= kHistBins) { b = kHistBins - 1; }
  return b;
}

template <typename T, typename Op>
__device__ __forceinline__ T tree256(T* a, T mine, Op op)
{
  const int t = threadIdx.x;
  a[t] = mine;
  __syncthreads();
  for (int s = kHistThreads >> 1; s > 0; s >>= 1) {
    if (t < s) { a[t] = op(a[t], a[t + s]); }
    __syncthreads();
  }
  const T r = a[0];
  __syncthreads();
  return r;
}

__global__ __launch_bounds__(kHistThreads) void sample_hist_max_kernel(
    const uint16_t* __restrict__ logits, float* __restrict__ slab_max, int V, int slab, float rep, float pres,
    const uint8_t* __restrict__ seen)
{
  __shared__ float tg[kHistThreads];
  const int lo = blockIdx.x * slab;
  const int hi = lo + slab < V ? lo + slab : V;
  float m = -INFINITY;
  for (int i = lo + threadIdx.x; i < hi; i += kHistThreads) {
    const float e = sample_eff(bf16_bits_to_f32(logits[i]), seen[i] != 0, rep, pres);
    m = e > m ? e : m;
  }
  const float r = tree256(tg, m, [](float a, float b) { return a > b ? a : b; });
  if (threadIdx.x == 0) { slab_max[blockIdx.x] = r; }
}

__global__ __launch_bounds__(kHistThreads) void sample_hist_weights_kernel(
    const uint16_t* __restrict__ logits, uint16_t* __restrict__ ws, const float* __restrict__ slab_max,
    float* __restrict__ partials, int V, int slab, int n_slabs, float temp, float rep, float pres,
    const uint8_t* __restrict__ seen)
{
  __shared__ float tg[kHistThreads];
  __shared__ uint32_t h_cnt[kHistBins];
  __shared__ uint32_t h_mass[kHistBins];
  const int t = threadIdx.x;
  auto fmax_op = [](float a, float b) { return a > b ? a : b; };
  float m = -INFINITY;
  for (int p = t; p < n_slabs; p += kHistThreads) { m = fmax_op(m, slab_max[p]); }
  const float maxl = tree256(tg, m, fmax_op);
  for (int b = t; b < kHistBins; b += kHistThreads) { h_cnt[b] = 0u; h_mass[b] = 0u; }
  __syncthreads();
  const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
  const int lo = blockIdx.x * slab;
  const int hi = lo + slab < V ? lo + slab : V;
  float z = 0.0f;
  for (int i = lo + t; i < hi; i += kHistThreads) {
    const float e = sample_eff(bf16_bits_to_f32(logits[i]), seen[i] != 0, rep, pres);
    const float w = sample_exp((e - maxl) * inv_t);
    ws[i] = (uint16_t)f32_to_bf16_bits(w);
    z = z + w;
    const int b = sample_bin(w);
    atomicAdd(&h_cnt[b], 1u);
    atomicAdd(&h_mass[b], (uint32_t)(w * 65536.0f));
  }
  const float Zs = tree256(tg, z, [](float a, float b) { return a + b; });     // its barriers also close the histogram
  float* P = partials + (size_t)blockIdx.x * (size_t)(2 * kHistBins + 1);
  for (int b = t; b < kHistBins; b += kHistThreads) {
    P[b] = (float)h_cnt[b];
    P[kHistBins + b] = (float)h_mass[b] * (1.0f / 65536.0f);
  }
  if (t == 0) { P[2 * kHistBins] = Zs; }
}

// One workgroup of 1024 threads: the slabs' histograms and Z added in slab order (a thread owns a cell; its loads
// are issued sixteen at a time, the additions stay in slab order), then the reference's scan
// (gpu-kernels/metal/ops/llm_elementwise.metal:3476-3497): one thread walks the bins from 0 with one running count
// and one running mass -- the same additions in the same order, so that a crossing at a knife edge falls into the
// same bin -- and stops at the bin where both targets are met (the bins are read eight at a time ahead of the
// additions; a full walk of 1024 bins, no filter ever met, is a few microseconds).
__global__ __launch_bounds__(kSampleThreads) void sample_hist_thresh_kernel(
    const float* __restrict__ partials, float* __restrict__ hist_out, float* __restrict__ wt_out, int n_slabs, int V,
    float top_p, int top_k, float min_p)
{
  __shared__ float hist[2 * kHistBins + 1];
  const int stride = 2 * kHistBins + 1;
  for (int c = threadIdx.x; c < stride; c += kSampleThreads) {
    float acc = 0.0f;
    for (int p0 = 0; p0 < n_slabs; p0 += 16) {
      float v[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) { v[q] = p0 + q < n_slabs ? partials[(size_t)(p0 + q) * stride + c] : 0.0f; }
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        if (p0 + q < n_slabs) { acc = acc + v[q]; }
      }
    }
    hist[c] = acc;
    hist_out[c] = acc;
  }
  __syncthreads();
  if (threadIdx.x != 0) { return; }
  const float target = top_p * hist[2 * kHistBins];
  float t_k = 0.0f, t_p = 0.0f, cum_cnt = 0.0f, cum_mass = 0.0f;
  bool have_k = false, have_p = false, done = false;
  const bool do_k = top_k > 0 && top_k < V;
  for (int b0 = 0; b0 < kHistBins && !done; b0 += 8) {
    float c8[8], m8[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) { c8[q] = hist[b0 + q]; m8[q] = hist[kHistBins + b0 + q]; }
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      if (!done) {
        cum_cnt = cum_cnt + c8[q];
        cum_mass = cum_mass + m8[q];
        if (do_k && !have_k && cum_cnt >= (float)top_k) { t_k = sample_exp(0.0f - (float)(b0 + q + 1) * kHistBinWidth); have_k = true; }
        if (!have_p && cum_mass >= target) { t_p = sample_exp(0.0f - (float)(b0 + q + 1) * kHistBinWidth); have_p = true; }
        done = (!do_k || have_k) && have_p;
      }
    }
  }
  wt_out[0] = fmaxf(fmaxf(t_k, fmaxf(min_p, 0.0f)), t_p);
}

__global__ __launch_bounds__(kHistThreads) void sample_hist_pick_kernel(
    const uint16_t* __restrict__ logits, const uint16_t* __restrict__ ws, const float* __restrict__ wt_in,
    float* __restrict__ pick_score, int32_t* __restrict__ pick_idx, int V, int slab, float temp, uint32_t seed, float rep,
    float pres, const uint8_t* __restrict__ seen)
{
  __shared__ float tg[kHistThreads];
  __shared__ int tgi[kHistThreads];
  const int t = threadIdx.x;
  const float inv_t = 1.0f / fmaxf(temp, 1e-6f);
  const float wt = wt_in[0];
  const int lo = blockIdx.x * slab;
  const int hi = lo + slab < V ? lo + slab : V;
  float best = -INFINITY;
  int bi = -1;
  for (int i = lo + t; i < hi; i += kHistThreads) {
    if (bf16_bits_to_f32(ws[i]) >= wt) {
      const float e = sample_eff(bf16_bits_to_f32(logits[i]), seen[i] != 0, rep, pres);
      const float u = sample_hash_u01(seed ^ ((uint32_t)i * 2654435761u + 1u));
      const float a = 0.0f - sample_log(u + 1e-20f) + 1e-20f;
      const float g = 0.0f - sample_log(a);
      const float score = e * inv_t + g;
      if (score > best) { best = score; bi = i; }
    }
  }
  tg[t] = best;
  tgi[t] = bi;
  __syncthreads();
  for (int s = kHistThreads >> 1; s > 0; s >>= 1) {
    if (t < s) {
      const bool take = tg[t + s] > tg[t] || (tg[t + s] == tg[t] && tgi[t + s] >= 0 && (tgi[t] < 0 || tgi[t + s] < tgi[t]));
      if (take) { tg[t] = tg[t + s]; tgi[t] = tgi[t + s]; }
    }
    __syncthreads();
  }
  if (t == 0) { pick_score[blockIdx.x] = tg[0]; pick_idx[blockIdx.x] = tgi[0]; }
}

__global__ __launch_bounds__(kHistThreads) void sample_hist_pick_combine_kernel(
    const float* __restrict__ pick_score, const int32_t* __restrict__ pick_idx, int n_slabs, int32_t* __restrict__ out_id,
    uint8_t* __restrict__ seen)
{
  __shared__ float tg[kHistThreads];
  __shared__ int tgi[kHistThreads];
  const int t = threadIdx.x;
  float best = -INFINITY;
  int bi = -1;
  for (int p = t; p < n_slabs; p += kHistThreads) {
    const float sc = pick_score[p];
    const int id = pick_idx[p];
    if (id < 0) { continue; }
    if (sc > best || (sc == best && (bi < 0 || id < bi))) { best = sc; bi = id; }
  }
  tg[t] = best;
  tgi[t] = bi;
  __syncthreads();
  for (int s = kHistThreads >> 1; s > 0; s >>= 1) {
    if (t < s) {
      const bool take = tgi[t + s] >= 0 && (tgi[t] < 0 || tg[t + s] > tg[t] || (tg[t + s] == tg[t] && tgi[t + s] < tgi[t]));
      if (take) { tg[t] = tg[t + s]; tgi[t] = tgi[t + s]; }
    }
    __syncthreads();
  }
  if (t == 0) {
    const int pick = tgi[0] >= 0 ? tgi[0] : 0;
    out_id[0] = pick;
    seen[pick] = 1;
  }
}

}  // namespace

size_t sample_hist_work_words(int n_slabs)
{
  return (size_t)n_slabs + (size_t)n_slabs * (2 * kHistBins + 1) + (2 * kHistBins + 1) + 1 + 2 * (size_t)n_slabs;
}

hipError_t launch_sample_hist(hipStream_t st, const uint16_t* logits, int32_t* out_id, int V, float temp, float top_p,
                              uint32_t seed, uint16_t* ws, float rep, float pres, int top_k, float min_p, uint8_t* seen,
                              int n_slabs, float* work)
{
  const int slab = (V + n_slabs - 1) / n_slabs;
  float* slab_max = work;
  float* partials = slab_max + n_slabs;
  float* hist = partials + (size_t)n_slabs * (2 * kHistBins + 1);
  float* wt = hist + (2 * kHistBins + 1);
  float* pick_score = wt + 1;
  int32_t* pick_idx = reinterpret_cast<int32_t*>(pick_score + n_slabs);
  const dim3 slabs((unsigned)n_slabs), one(1), block(kHistThreads);
  hipError_t e = launch_kernel(sample_hist_max_kernel, slabs, block, 0, st, logits, slab_max, V, slab, rep, pres,
                               (const uint8_t*)seen);
  if (e != hipSuccess) { return e; }
  e = launch_kernel(sample_hist_weights_kernel, slabs, block, 0, st, logits, ws, (const float*)slab_max, partials, V, slab,
                    n_slabs, temp, rep, pres, (const uint8_t*)seen);
  if (e != hipSuccess) { return e; }
  e = launch_kernel(sample_hist_thresh_kernel, one, dim3(kSampleThreads), 0, st, (const float*)partials, hist, wt, n_slabs, V,
                    top_p, top_k, min_p);
  if (e != hipSuccess) { return e; }
  e = launch_kernel(sample_hist_pick_kernel, slabs, block, 0, st, logits, (const uint16_t*)ws, (const float*)wt, pick_score,
                    pick_idx, V, slab, temp, seed, rep, pres, (const uint8_t*)seen);
  if (e != hipSuccess) { return e; }
  return launch_kernel(sample_hist_pick_combine_kernel, one, block, 0, st, (const float*)pick_score,
                       (const int32_t*)pick_idx, n_slabs, out_id, seen);
}

hipError_t launch_sample_topp(hipStream_t st, const uint16_t* logits, int32_t* out_id, int V, float temp, float top_p,
                              uint32_t seed, uint16_t* ws, int n_iter, float rep, float pres, int top_k, float min_p,
                              uint8_t* seen)
{
  return launch_kernel(sample_topp_kernel, dim3(1), dim3(kSampleThreads), 0, st, logits, out_id, V, temp, top_p, seed, ws,
                       n_iter, rep, pres, top_k, min_p, seen);
}

}  // namespace vpq

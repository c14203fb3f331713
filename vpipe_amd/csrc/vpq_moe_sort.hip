// Counting sort of the (token, expert) pairs of an MoE block into per-expert blocks of slots, each
// expert's share padded to whole blocks of `block_rows` slots -- the row order the grouped expert GEMM
// multiplies in (gpu-kernels/metal/ops/llm_elementwise.metal:255-326: moe_ifill_i32, moe_hist_i32,
// moe_sort_setup_i32, moe_scatter_i32; driven by
// generative-models/qwen3/metal-qwen-model.cc:4213-4237).
//
//   tile2e[t]  expert of block t, -1 for a block no expert uses;
//   srow[i]    x (token) row of slot i = pair / top_k, -1 for a padding slot;
//   sdst[i]    the pair of slot i, -1 for a padding slot;
//   ntiles[0]  blocks in use.
// Experts come in ascending order, expert e's first slot is block_rows * (blocks of the experts below
// it).  The order of the pairs inside an expert's share is whatever order their atomic tickets come
// in; every consumer treats the slots independently, so results do not depend on it.  A pair whose
// expert id lies outside [0, n_experts) gets no slot.
//
// Four small launches on the caller's stream (no allocation; ws holds 3 n_experts ints): fill, histogram,
// offsets by one wavefront (a scan over the experts), scatter.
#include "vpq_device.h"
#include "vpq_internal.h"

namespace vpq {

namespace {

__global__ __launch_bounds__(256) void moe_sort_fill_kernel(int* tile2e, int max_tiles, int* srow, int* sdst, int npad,
                                                            int* hist, int n_experts)
{
  const int stride = (int)gridDim.x * 256;
  const int cover = npad > n_experts ? npad : n_experts;     // max_tiles <= npad
  for (int i = (int)blockIdx.x * 256 + (int)threadIdx.x; i < cover; i += stride) {
    if (i < npad) {
      srow[i] = -1;
      sdst[i] = -1;
    }
    if (i < max_tiles) { tile2e[i] = -1; }
    if (i < n_experts) { hist[i] = 0; }
  }
}

// Pairs per workgroup of the histogram and scatter kernels, and the expert count up to which a workgroup
// counts in LDS first (one global atomic per expert and workgroup instead of one per pair).
constexpr int kSortChunk = 1024;
constexpr int kSortLdsExperts = 4096;

__global__ __launch_bounds__(256) void moe_sort_hist_kernel(const int* __restrict__ eid, int n_pairs, int n_experts, int* hist)
{
  __shared__ int local[kSortLdsExperts];
  const int p0 = (int)blockIdx.x * kSortChunk;
  const bool in_lds = n_experts <= kSortLdsExperts;
  if (in_lds) {
    for (int e = (int)threadIdx.x; e < n_experts; e += 256) { local[e] = 0; }
    __syncthreads();
  }
  for (int i = (int)threadIdx.x; i < kSortChunk; i += 256) {
    const int p = p0 + i;
    if (p >= n_pairs) { break; }
    const int e = eid[p];
    if (e >= 0 && e < n_experts) { atomicAdd(in_lds ? local + e : hist + e, 1); }
  }
  if (in_lds) {
    __syncthreads();
    for (int e = (int)threadIdx.x; e < n_experts; e += 256) {
      if (local[e] != 0) { atomicAdd(hist + e, local[e]); }
    }
  }
}

// One wavefront: lane l owns the experts [l * per, (l + 1) * per).
__global__ __launch_bounds__(64) void moe_sort_setup_kernel(const int* __restrict__ hist, int* boff, int* cursor, int* tile2e,
                                                            int* ntiles, int n_experts, int block_rows, int max_tiles)
{
  const int lane = (int)threadIdx.x;
  const int per = (n_experts + 63) / 64;
  const int e0 = lane * per;
  int mine = 0;                                   // blocks of this lane's experts
  for (int i = 0; i < per; ++i) {
    const int e = e0 + i;
    if (e < n_experts) { mine += (hist[e] + block_rows - 1) / block_rows; }
  }
  int incl = mine;                                // inclusive scan over the lanes
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = __shfl_up(incl, d, 64);
    if (lane >= d) { incl += up; }
  }
  int t = incl - mine;                            // first block of this lane's experts
  for (int i = 0; i < per; ++i) {
    const int e = e0 + i;
    if (e >= n_experts) { break; }
    const int nb = (hist[e] + block_rows - 1) / block_rows;
    boff[e] = t * block_rows;
    cursor[e] = 0;
    for (int j = 0; j < nb; ++j) {
      if (t + j < max_tiles) { tile2e[t + j] = e; }
    }
    t += nb;
  }
  if (lane == 63) { ntiles[0] = incl; }
}

__global__ __launch_bounds__(256) void moe_sort_scatter_kernel(const int* __restrict__ eid, const int* __restrict__ boff,
                                                               int* cursor, int* srow, int* sdst, int n_pairs, int top_k,
                                                               int n_experts, int npad)
{
  __shared__ int local[kSortLdsExperts];     // pairs of this workgroup per expert, then their first ticket
  const int p0 = (int)blockIdx.x * kSortChunk;
  const bool in_lds = n_experts <= kSortLdsExperts;
  int rank[kSortChunk / 256];
  if (in_lds) {
    for (int e = (int)threadIdx.x; e < n_experts; e += 256) { local[e] = 0; }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kSortChunk / 256; ++j) {
      const int p = p0 + j * 256 + (int)threadIdx.x;
      const int e = p < n_pairs ? eid[p] : -1;
      rank[j] = (e >= 0 && e < n_experts) ? atomicAdd(local + e, 1) : 0;
    }
    __syncthreads();
    for (int e = (int)threadIdx.x; e < n_experts; e += 256) {
      const int c = local[e];
      if (c != 0) { local[e] = atomicAdd(cursor + e, c); }     // a run of c tickets
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < kSortChunk / 256; ++j) {
    const int p = p0 + j * 256 + (int)threadIdx.x;
    if (p >= n_pairs) { continue; }
    const int e = eid[p];
    if (e < 0 || e >= n_experts) { continue; }
    const int ticket = in_lds ? local[e] + rank[j] : atomicAdd(cursor + e, 1);
    const int slot = boff[e] + ticket;
    if (slot < npad) {
      srow[slot] = p / top_k;
      sdst[slot] = p;
    }
  }
}

// `moe_scatter_back_f16` (gpu-kernels/metal/ops/llm_elementwise.metal:328-342): rows of the sorted down
// projection back to pair order, partials[sdst[slot]] = dsorted[slot]; padding slots (sdst < 0) and destinations
// outside [0, n_pairs) are skipped.  16 bytes per thread where the rows allow, else 2.
template <typename V>
__global__ __launch_bounds__(256) void moe_scatter_back_kernel(const V* __restrict__ dsorted, const int* __restrict__ sdst,
                                                              V* __restrict__ partials, int npad, int row_vecs, int n_pairs)
{
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)npad * (size_t)row_vecs) { return; }
  const int slot = (int)(i / (size_t)row_vecs);
  const int v = (int)(i - (size_t)slot * (size_t)row_vecs);
  const int p = sdst[slot];
  if (p < 0 || p >= n_pairs) { return; }
  partials[(size_t)p * row_vecs + v] = dsorted[(size_t)slot * row_vecs + v];
}

}  // namespace

hipError_t launch_moe_scatter_back(hipStream_t st, const uint16_t* dsorted, const int* sdst, uint16_t* partials, int npad,
                                   int H, int n_pairs, bool wide)
{
  if (wide) {
    const size_t n = (size_t)npad * (size_t)(H / 8);
    return launch_kernel(moe_scatter_back_kernel<uint4>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                         reinterpret_cast<const uint4*>(dsorted), sdst, reinterpret_cast<uint4*>(partials), npad, H / 8, n_pairs);
  }
  const size_t n = (size_t)npad * (size_t)H;
  return launch_kernel(moe_scatter_back_kernel<uint16_t>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, dsorted, sdst,
                       partials, npad, H, n_pairs);
}

hipError_t launch_moe_sort(hipStream_t st, const int* pair_eid, int n_pairs, int top_k, int n_experts, int block_rows,
                           int max_tiles, int* tile2e, int* srow, int* sdst, int* ntiles, int* ws)
{
  const int npad = max_tiles * block_rows;
  int* hist = ws;
  int* boff = ws + n_experts;
  int* cursor = ws + 2 * n_experts;
  const int cover = npad > n_experts ? npad : n_experts;
  int fill_blocks = (cover + 255) / 256;
  if (fill_blocks > 1024) { fill_blocks = 1024; }
  hipError_t e = launch_kernel(moe_sort_fill_kernel, dim3((unsigned)fill_blocks), dim3(256), 0, st, tile2e, max_tiles, srow,
                               sdst, npad, hist, n_experts);
  if (e != hipSuccess) { return e; }
  const dim3 pgrid((unsigned)((n_pairs + kSortChunk - 1) / kSortChunk));
  e = launch_kernel(moe_sort_hist_kernel, pgrid, dim3(256), 0, st, pair_eid, n_pairs, n_experts, hist);
  if (e != hipSuccess) { return e; }
  e = launch_kernel(moe_sort_setup_kernel, dim3(1), dim3(64), 0, st, (const int*)hist, boff, cursor, tile2e, ntiles,
                    n_experts, block_rows, max_tiles);
  if (e != hipSuccess) { return e; }
  return launch_kernel(moe_sort_scatter_kernel, pgrid, dim3(256), 0, st, pair_eid, (const int*)boff, cursor, srow, sdst,
                       n_pairs, top_k, n_experts, npad);
}

}  // namespace vpq

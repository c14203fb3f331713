// Host-side launch functions behind the C ABI.  Each validates nothing: the
// C ABI layer (vpq_api.hip) has already checked shapes, alignment and pointers.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>
#include <stdint.h>

#include <string>
#include <cstring>
#include <vector>

namespace vpq {

// Measurement aid: while `on`, every kernel launch is bracketed by a pair of HIP
// events handed to hipExtLaunchKernel, which stamps them at the kernel's own
// start and end (no launch gap included).  One state per process; the
// benchmark enables it from a single thread.
struct ProfileState {
  bool on = false;
  std::vector<hipEvent_t> events;  // start0, stop0, start1, stop1, ...
  size_t used = 0;
};
ProfileState& profile_state();

template <typename F, typename... Args>
inline hipError_t launch_kernel(F kernel, dim3 grid, dim3 block, size_t lds_bytes, hipStream_t st,
                                Args... args)
{
  ProfileState& ps = profile_state();
  if (ps.on && ps.used + 2 <= ps.events.size()) {
    hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, st, ps.events[ps.used],
                          ps.events[ps.used + 1], 0, args...);
    ps.used += 2;
  } else {
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, st, args...);
  }
  return hipGetLastError();
}

// Kernel arguments in registers at wavefront start.  The library is compiled with kernel-argument preloading: the
// first fourteen 32-bit words of a kernel's arguments arrive in scalar registers with the wavefront instead of
// being loaded from the argument buffer (a round trip of most of a microsecond before the first request can go
// out) -- but only if they are scalar arguments; an aggregate argument is always read from the buffer.  A kernel
// that takes a parameter struct P therefore takes its first 56 bytes as fourteen words (VPQ_PRELOADED_WORDS) and the
// rest as PreloadTail<P>, and puts P together again with preload_assemble; launch_preloaded splits P on the host.
// Order the fields of P so that what the first requests need comes first and what only the store needs comes last.
constexpr int kPreloadWords = 14;
template <typename P>
struct PreloadTail {
  static_assert(sizeof(P) > kPreloadWords * 4 && sizeof(P) % 4 == 0, "parameter struct of whole words, longer than the preloaded part");
  uint32_t w[(sizeof(P) - kPreloadWords * 4) / 4];
};
#define VPQ_PRELOADED_WORDS                                                                                          \
  uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, uint32_t a4, uint32_t a5, uint32_t a6, uint32_t a7, uint32_t a8, \
      uint32_t a9, uint32_t a10, uint32_t a11, uint32_t a12, uint32_t a13
#define VPQ_PRELOADED_WORD_LIST a0, a1, a2, a3, a4, a5, a6, a7, a8, a9, a10, a11, a12, a13

template <typename P>
__device__ __forceinline__ P preload_assemble(VPQ_PRELOADED_WORDS, const PreloadTail<P>& tail)
{
  const uint32_t head[kPreloadWords] = {VPQ_PRELOADED_WORD_LIST};
  P p;
  __builtin_memcpy(&p, head, sizeof(head));
  __builtin_memcpy(reinterpret_cast<char*>(&p) + sizeof(head), tail.w, sizeof(tail.w));
  return p;
}

template <typename F, typename P>
inline hipError_t launch_preloaded(F kernel, dim3 grid, dim3 block, size_t lds_bytes, hipStream_t st, const P& p)
{
  uint32_t h[kPreloadWords];
  PreloadTail<P> tail;
  std::memcpy(h, &p, sizeof(h));
  std::memcpy(tail.w, reinterpret_cast<const char*>(&p) + sizeof(h), sizeof(tail.w));
  return launch_kernel(kernel, grid, block, lds_bytes, st, h[0], h[1], h[2], h[3], h[4], h[5], h[6], h[7], h[8], h[9], h[10],
                       h[11], h[12], h[13], tail);
}

// Measurement aids (vpq_profile.hip): a kernel that does nothing, a kernel that only reads `bytes` of src.
hipError_t launch_profile_empty(hipStream_t st, uint32_t* sink);
hipError_t launch_profile_read(hipStream_t st, const void* src, size_t bytes, uint32_t* sink);

// QmvArgs::gate_act beyond the pair activations (1 SwiGLU, 2 GEGLU): y[n] = elt(gelu_tanh(elt(sum[n])) * mul[n]),
// the fused per-layer-input gate `affine_qmv_gelu_mul_w4g64` (gpu-kernels/metal/quant/affine_qmv.metal:751-768); the
// multiplier [N] travels in `residual`.  One row of x, element-typed store only.
constexpr int kStoreGeluMul = 3;
// qmv_rows8_kernel, ungated: y = elt(sigmoid(sum)), the shared-expert gate `affine_moe_gate_w8g64`
// (gpu-kernels/metal/quant/affine_qmv.metal:1323-1349).
constexpr int kStoreSigmoid = 4;

struct QmvArgs {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  const uint16_t* x;
  void* y;                   // bf16 [M,N] or fp32 [M,N]
  const uint16_t* residual;  // nullable, bf16 [M,N]
  int K, N, M;
  bool y_f32;
  void* ws;                  // split-K scratch (nullable)
  size_t ws_bytes;
  int cu_count;
  // Non-zero (1 SwiGLU, 2 GEGLU): the pack is an interleaved gate|up matrix (row 2g gate, 2g+1 up;
  // N even) and y is [M, N/2] = act(gate) * up.  No residual with it.
  int gate_act = 0;
};

struct GemmArgs {
  const uint32_t* w;         // packed codes
  const uint16_t* scales;
  const uint16_t* biases;
  const uint16_t* x;         // [M,K]
  uint16_t* y;               // [M,N]
  int K, N, M;
  const uint16_t* lora_t;    // nullable, [M,r]
  const uint16_t* lora_b;    // nullable, [N,r]
  int r;
  int cu_count;
  // Non-zero (1 SwiGLU, 2 GEGLU): interleaved gate|up pack,
  // y[m * out_stride + out_off + g] = act(gate) * up, g < N/2.
  int gate_act = 0;
  int out_stride = 0;
  int out_off = 0;
  int bits = 4;              // 8: one byte per value, w [N, K/4]
  int group = 64;            // 32: scales / biases [N, K/32] (4-bit only)
  bool f16 = false;          // elements are IEEE binary16 (the large-tile kernel only, no adapter)
};

hipError_t launch_dequant(hipStream_t st, const uint32_t* w, const uint16_t* scales,
                          const uint16_t* biases, uint16_t* out, int K, int N);
// out[t, :] = dense expansion of table row ids[t] (zeros for an id outside [0, vocab)).
hipError_t launch_embed_gather(hipStream_t st, const int* ids, const uint32_t* w, const uint16_t* scales,
                               const uint16_t* biases, uint16_t* out, int H, int T, int vocab);
hipError_t launch_qmv_simple(hipStream_t st, const QmvArgs& a);
// group-32 twins (scales, biases [N, K/32]; K % 32 == 0); scale_only: Q4_0 pack, bias = -8 * scale, a.biases unread.
hipError_t launch_dequant_g32(hipStream_t st, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                              uint16_t* out, int K, int N);
hipError_t launch_qmv_simple_g32(hipStream_t st, const QmvArgs& a, bool scale_only);
hipError_t launch_qmv_rows_g32(hipStream_t st, const QmvArgs& a, bool scale_only);   // M <= 2
// The 8-bit twins (one byte per value, w is [N, K/4] words): dense expansion and the general QMV kernel.
hipError_t launch_dequant8(hipStream_t st, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           uint16_t* out, int K, int N, int group = 64, bool f16 = false);
hipError_t launch_qmv_simple8(hipStream_t st, const QmvArgs& a, int group = 64);
// 8-bit group-64 pack -> 4-bit group-64 pack of the same shape (one thread per group).
hipError_t launch_requant_w8_to_w4(hipStream_t st, const uint32_t* w8, const uint16_t* s8, const uint16_t* b8,
                                   uint32_t* w4, uint16_t* s4, uint16_t* b4, int K, int N);
// Mixed-width fused gate/up over separate packs (4 or 8 bits each); rows = pairs (pair_eid) or rows of x.
struct SplitGateUp {
  const uint32_t* wg; const uint16_t* sg; const uint16_t* bg; int gate_bits;
  const uint32_t* wu; const uint16_t* su; const uint16_t* bu; int up_bits;
  const uint16_t* x; uint16_t* y;
  int K, F, rows, gate_act;
  const int* pair_eid; int x_div, n_experts;
};
hipError_t launch_qmv_split_gate_up(hipStream_t st, const SplitGateUp& a);
// 8-bit gated / gathered QMV, one wavefront per output and row (a.gate_act: interleaved gate|up pack);
// rows = rows of x, or with pair_eid the (token, expert) pairs over a batched pack.
hipError_t launch_qmv_rows8(hipStream_t st, const QmvArgs& a, int rows, const int* pair_eid, int x_div, int n_experts);
// Two-slot expert-sorted GEMV over a batched 8-bit pack (a.gate_act != 0: x rows gathered through srow).
hipError_t launch_qmv_rows8_sorted(hipStream_t st, const QmvArgs& a, const int* tile2e, const int* srow, int tiles,
                                   int n_experts);
// Returns hipErrorInvalidValue if the shape is outside what the MFMA kernel
// handles (the caller then falls back to the simple kernel).
bool qmv_mfma_supports(int K, int N, int M);
hipError_t launch_qmv_mfma(hipStream_t st, const QmvArgs& a);
// Up to four projections that share x, K and M in ONE launch (q|k|v, gate|up): a.w/scales/
// biases/y/N/residual/ws are ignored, the segments give them.
struct QmvSeg {
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  void* y;
  int N;
};
struct QmvGroup {
  int count;
  QmvSeg seg[4];
};
hipError_t launch_qmv_mfma_group(hipStream_t st, const QmvArgs& a, const QmvGroup& g);
// Streaming kernel for M = 1 (K % 512 == 0, K >= 2048, 16-byte aligned scales / biases): one wavefront per
// (row set, K part), every load requested up front; also as one launch over up to four packs that share x.
bool qmv_flow_supports(int K, int N, int M);
hipError_t launch_qmv_flow(hipStream_t st, const QmvArgs& a);
hipError_t launch_qmv_flow_f16(hipStream_t st, const QmvArgs& a);    // IEEE binary16 elements
hipError_t launch_qmv_flow_group(hipStream_t st, const QmvArgs& a, const QmvGroup& g, bool f16 = false);
bool qmv_stream_supports(int K, int N, int M);
hipError_t launch_qmv_stream(hipStream_t st, const QmvArgs& a, bool f16 = false);
bool qmv_ring_supports(int K, int N, int M);
// tc_hint / nw_hint > 0 force the tiles / wavefronts per workgroup (measurement only).
hipError_t launch_qmv_ring(hipStream_t st, const QmvArgs& a, int tc_hint, int splits_hint, bool f16 = false);
size_t qmv_ring_workspace_bytes(int K, int N, int M);   // planes of the widest K split the ring kernel takes
// Row-streaming kernel (M <= 2, any K % 64): rows_per_wave in {2, 4}, 0 = default.
bool qmv_rows_supports(int K, int N, int M);
hipError_t launch_qmv_rows(hipStream_t st, const QmvArgs& a, int rows_per_wave);
// out[m, k] = bf16(x[m, k] * rsqrt(mean(x[m, :]^2) + eps) * norm_w[k]): the RMSNorm ahead of the fused-QKV GEMV.
hipError_t launch_rmsnorm(hipStream_t st, const uint16_t* x, const uint16_t* norm_w, uint16_t* out, int K, int M, float eps);
hipError_t launch_qmv_rows_group(hipStream_t st, const QmvArgs& a, const QmvGroup& g, int group = 64,
                                 bool scale_only = false);
// Gathered (MoE) form, M = 1 per pair: a.w/scales/biases are batches [E, N, ...] of expert slabs,
// pair p contracts slab pair_eid[p] with x row p / x_div into y row p (zeros for an id outside
// [0, n_experts)); a.gate_act as in the plain form.
hipError_t launch_qmv_rows_gather(hipStream_t st, const QmvArgs& a, const int* pair_eid, int pairs, int x_div,
                                  int n_experts);
// Sorted pairs, two slots per tile (a.M = 2): expert tile2e[tile], x row srow[slot] (x_from_srow) or the slot.
hipError_t launch_qmv_rows_sorted(hipStream_t st, const QmvArgs& a, const int* tile2e, const int* srow, int tiles,
                                  bool x_from_srow, int n_experts);
// Greedy argmax of `rows` rows of V bf16 logits (lowest index among equal maxima, a NaN never
// wins): one workgroup per row, or slabs into `partials` (two 4-byte slots per slab: value, index)
// and a combine; argmax_parts(V) is the slab count the size-based entrance uses.
int argmax_parts(int V);
// Rows the static scratch of vpq_argmax_bf16_static holds, and its per-device address (resolved once per
// device, with that device current; allocates nothing).
constexpr int kArgmaxStaticRows = 64;
hipError_t argmax_static_scratch(float** out);
hipError_t launch_argmax_row(hipStream_t st, const uint16_t* logits, int* out_id, int V, int rows);
hipError_t launch_argmax_partial(hipStream_t st, const uint16_t* logits, float* partials, int V, int rows, int parts);
hipError_t launch_argmax_combine(hipStream_t st, const float* partials, int* out_id, int rows, int parts);
// t[M,r] = bf16(alpha * bf16(x . A^T)), r in {32, 64, 96, 128}.
// Adapter ranks: multiples of 16 up to this (the reference runs 16 and measures 384).
constexpr int kLoraMaxRank = 512;
hipError_t launch_lora_a(hipStream_t st, const uint16_t* x, const uint16_t* a, uint16_t* t, int M, int K, int r,
                         float alpha, bool f16 = false);
// 256x128-tile quantized GEMM (+ fused LoRA second factor); a.w must be non-null.
hipError_t launch_qmm_tile(hipStream_t st, const GemmArgs& a);
// Grouped (expert-sorted) form of the tile kernel at 128 rows per block: a.w/scales/biases are the
// batched pack [E, N, ...], a.M the padded slot count (a multiple of kGroupedBlockRows); see TileParams.
constexpr int kGroupedBlockRows = 128;
struct GroupedArgs {
  const int* tile2e;   // [a.M / kGroupedBlockRows]
  const int* srow;     // [a.M] or nullptr: x row per slot
  const int* sdst;     // [a.M] or nullptr: y row per slot
  int n_experts, rows_x, rows_y;
};
hipError_t launch_moe_scatter_back(hipStream_t st, const uint16_t* dsorted, const int* sdst, uint16_t* partials, int npad,
                                   int H, int n_pairs, bool wide);
hipError_t launch_moe_sort(hipStream_t st, const int* pair_eid, int n_pairs, int top_k, int n_experts, int block_rows,
                           int max_tiles, int* tile2e, int* srow, int* sdst, int* ntiles, int* ws);
hipError_t launch_qmm_grouped(hipStream_t st, const GemmArgs& a, const GroupedArgs& g);
// Large-tile kernel (256 x 256 or 256 x 192 per workgroup, four wavefronts that each load, dequantize
// and multiply): K % 512 == 0, 16-byte aligned scales / biases, no gated store; same bits as the tile
// kernel.  tile_n 0 = qmm_big_tile_n().
bool qmm_big_supports(const GemmArgs& a);
int qmm_big_tile_n(int N, int M, int cu_count, int max_width = 256, bool with_192 = true);
hipError_t launch_qmm_big(hipStream_t st, const GemmArgs& a, int tile_n);
// Split-K form of the same kernel (no adapter, no gated store): `splits` shares of the K steps,
// fp32 planes [splits][M][N] in `plane`, then a fold.  qmm_choose_splits() returns 1 where the tiles
// alone fill the chip.
int qmm_choose_splits(int K, int N, int M, int cu_count);
size_t qmm_splitk_workspace_bytes(int K, int N, int M, int cu_count);
hipError_t launch_qmm_tile_splitk(hipStream_t st, const GemmArgs& a, int splits, float* plane);
// y[M,N] = x[M,K] . b[N,K]^T on the large-tile kernel with dense 2-byte weights (bf16, or binary16 with f16;
// fp32 accumulate, one rounding).  0, or -2 (shape outside the kernel / launch failed) with *why set.
bool dense_gemm_supports(int M, int N, int K);
hipError_t launch_dense_gemm(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K,
                             bool f16, int cu_count, const uint16_t* lora_t = nullptr, const uint16_t* lora_b = nullptr,
                             int r = 0);
int dense_gemm_bf16(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K, int cu_count,
                    std::string* why);
int dense_gemm_elt(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K, bool f16,
                   int cu_count, std::string* why, const uint16_t* lora_t = nullptr, const uint16_t* lora_b = nullptr,
                   int r = 0);
// IEEE binary16 element type (the reference's VPIPE_ELT = half build): dense expansion and the general QMV.
hipError_t launch_dequant_f16(hipStream_t st, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                              uint16_t* out, int K, int N);
hipError_t launch_qmv_simple_f16(hipStream_t st, const QmvArgs& a);
hipError_t launch_quantize(hipStream_t st, const uint16_t* src, uint32_t* w, uint16_t* s_f16,
                           uint16_t* b_f16, int K, int N, float clip, int bits = 4, int group = 64, bool f16_src = false);
hipError_t launch_f16_to_bf16(hipStream_t st, const uint16_t* in, uint16_t* out, size_t count);
// out row 2i = a row i, out row 2i+1 = b row i; rows of row_bytes (a multiple of 2) bytes.
hipError_t launch_interleave_rows(hipStream_t st, const void* a, const void* b, void* out, size_t row_bytes,
                                  size_t rows);

// The sampler tail (vpq_sample.hip): one workgroup over one row of logits.
hipError_t launch_sample_topp(hipStream_t st, const uint16_t* logits, int32_t* out_id, int V, float temp, float top_p,
                              uint32_t seed, uint16_t* ws, int n_iter, float rep, float pres, int top_k, float min_p,
                              uint8_t* seen);
// The sampler over n_slabs workgroups with histogram thresholds; work holds sample_hist_work_words(n_slabs) fp32 words.
size_t sample_hist_work_words(int n_slabs);
hipError_t launch_sample_hist(hipStream_t st, const uint16_t* logits, int32_t* out_id, int V, float temp, float top_p,
                              uint32_t seed, uint16_t* ws, float rep, float pres, int top_k, float min_p, uint8_t* seen,
                              int n_slabs, float* work);

}  // namespace vpq

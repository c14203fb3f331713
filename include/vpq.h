/*
 * vpq.h -- C ABI of the MI355X (gfx950) 4-bit / group-64 affine quantized
 * linear operator: QMV (decode GEMV, 1..16 rows), QMM (prefill / DiT GEMM with
 * an optional fused runtime LoRA), the dense expansion of a pack, and the
 * packer.
 *
 * The entry points replace, one for one, the Metal kernels VPIPE's model
 * families dispatch through their quantized-linear convention
 * (docs/PLUGINS.md:202-224): the argument ORDER is the Metal buffer-slot order
 *     0:w  1:scales  2:biases  3:x  4:y  5:K  6:N  [7:M]
 * so a call site changes one line.  Citations are file:line in the reference
 * tree (tgo-app-dev/vpipe).
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer (hipMalloc / torch device memory).
 *   - bf16 values are uint16_t bit patterns.  Element type is bf16 everywhere
 *     (the reference's `_bf16` metallib twins, -DVPIPE_ELT=bfloat).
 *   - Packed layout, unchanged from generative-models/quantize:
 *       w       uint32 [N, K/8]    q[n, 8j+i] = (w[n,j] >> 4i) & 0xF
 *       scales  bf16   [N, K/64]
 *       biases  bf16   [N, K/64]   W[n,k] = scales[n,k/64]*q[n,k] + biases[n,k/64]
 *     `biases` is the quantizer's zero point, NOT the linear layer's additive
 *     bias; no kernel here has an additive-bias slot, as in the reference
 *     (generative-models/minimax-h3/metal-minimax-h3-transformer.cc:2250-2256).
 *   - Calls are asynchronous and ordered on `stream` (a hipStream_t passed as
 *     void*; NULL is the null stream).  They never synchronise and never
 *     allocate; scratch is caller-provided.  The caller owns every buffer and
 *     keeps it alive until the stream has passed the call.
 *   - Return value: VPQ_OK or a negative vpq_status.  Shape and alignment
 *     preconditions are checked on the host before anything is launched; a
 *     failed check launches nothing.  The reference leaves those checks to the
 *     caller (docs/PLUGINS.md:207-220) and reports GPU faults only at
 *     Fence::wait_ok (apple-silicon/metal-compute/command-stream.h:92-99); a
 *     fault here surfaces at the caller's next stream synchronisation.
 *   - A stream must not run two calls concurrently that share a workspace.
 */
#ifndef VPQ_H
#define VPQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* vpq_stream_t; /* hipStream_t */

typedef enum vpq_status {
  VPQ_OK = 0,
  VPQ_ERR_NULL_POINTER = -1,  /* a required buffer is NULL */
  VPQ_ERR_BAD_SHAPE = -2,     /* K, N, M, r out of the supported domain */
  VPQ_ERR_MISALIGNED = -3,    /* a pointer is not aligned as required */
  VPQ_ERR_WORKSPACE = -4,     /* workspace missing or too small */
  VPQ_ERR_DEVICE = -5,        /* the HIP runtime reported an error */
  VPQ_ERR_UNSUPPORTED = -6    /* not a gfx950 device */
} vpq_status;

/* Library version (major*10000 + minor*100 + patch). */
int vpq_version(void);

/* Human-readable text of a status code; never NULL. */
const char* vpq_status_string(int status);

/* Text of the last HIP error this thread saw inside the library ("" if none). */
const char* vpq_last_device_error(void);

/* Checks that the current HIP device is a gfx950 part and caches its
 * properties.  Optional: every entry point does it on first use.
 * Stands where MetalCompute::valid() stands
 * (apple-silicon/metal-compute/metal-compute.h:274-301). */
int vpq_init(void);

/* Number of compute units of the current device (0 before a successful init). */
int vpq_device_cu_count(void);

/* ---- a1: dense expansion ------------------------------------------------
 * Replaces `affine_dequant_w4g64`
 * (gpu-kernels/metal/quant/affine_dequant.metal:25-58; slots 0:w 1:scales
 * 2:biases 3:y_deq 4:K 5:N).  w_deq[n,k] = bf16_rne(fp32(s*q + b)), bit-exact
 * with the reference expression.  Requires K % 64 == 0, K, N > 0; w_deq
 * 16-byte aligned. */
int vpq_dequant_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, uint16_t* w_deq, int K, int N);

/* Dequantizing embedding gather over the same pack (a tied lm_head / embedding
 * table).  Replaces `dequant_embed_gather_f16`
 * (gpu-kernels/metal/ops/llm_elementwise.metal:1676-1701; slots 0:ids 1:w 2:scales
 * 3:biases 4:out 5:H, grid (H, T, 1)): out[t, :] = bf16_rne(fp32(s*q + b)) of table
 * row ids[t], bit-identical to that row of vpq_dequant_w4g64_bf16.  `ids` is a
 * device array of T int32; the table is [vocab, H].  A row whose id is outside
 * [0, vocab) is filled with zeros (the reference reads out of bounds there).
 * Requires H % 64 == 0, T > 0; out 16-byte aligned. */
int vpq_embed_gather_w4g64_bf16(vpq_stream_t stream, const int32_t* ids, const uint32_t* w,
                                const uint16_t* scales, const uint16_t* biases, uint16_t* out,
                                int H, int T, int vocab);

/* ---- a2/a3/a4: QMV, 1 <= M <= 16 ---------------------------------------
 * Replaces `affine_qmv_w4g64` (gpu-kernels/metal/quant/affine_qmv.metal:286-301;
 * slots 0:w 1:scales 2:biases 3:x 4:y 5:K 6:N), its `_add` twin (:347-363,
 * slot 7: residual) and the batched tiles `affine_qmv_batch*_w4g64`
 * (:1573-1709, 2156-2330; slot 7: m_total): y[M,N] = x[M,K] . W^T with the
 * QMV arithmetic -- the weight is never rounded to bf16; per (row, group) the
 * kernel forms sum(x*q) and sum(x) in fp32 and combines them as
 * scale*sum(x*q) + bias*sum(x) (affine_qmv.metal:151-174), fp32 accumulate,
 * one bf16 rounding on store.  With `residual` ([M,N] bf16, nullable) the
 * rounded result is added to it in fp32 and rounded again, as `_add` does
 * (:264-266).
 * Requires K % 64 == 0, N > 0, 1 <= M <= 16.
 * `ws` is scratch for the split of K across workgroups (fp32 planes):
 * vpq_qmv_workspace_bytes() bytes, 16-byte aligned, no initial content
 * needed; it may be NULL, in which case shapes that would have split K run
 * unsplit.
 * `variant`: 0 = automatic; other values select a specific kernel for
 * measurement (see VPQ_QMV_* below). */
int vpq_qmv_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* x, uint16_t* y,
                       int K, int N, int M, const uint16_t* residual,
                       void* ws, size_t ws_bytes, int variant);

/* Same arithmetic, fp32 [M,N] output before the final rounding (measurement of
 * the accumulation error apart from the bf16 store). */
int vpq_qmv_w4g64_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                         const uint16_t* biases, const uint16_t* x, float* y,
                         int K, int N, int M, void* ws, size_t ws_bytes, int variant);

/* Bytes of split-K scratch the QMV entry points may use for this shape
 * (an upper bound over variants; a multiple of 256). */
size_t vpq_qmv_workspace_bytes(int K, int N, int M);

enum {
  VPQ_QMV_AUTO = 0,
  VPQ_QMV_SIMPLE = 1,      /* one wavefront per output row, fp32 VALU */
  VPQ_QMV_MFMA = 2,        /* LDS-staged codes, bf16 MFMA on the integer codes */
  /* 3 is unassigned */
  VPQ_QMV_STREAM = 4,      /* M <= 4: persistent workgroups, x staged in LDS, prefetched items */
  VPQ_QMV_RING = 5,        /* x in registers across a workgroup's tiles, codes through a two-slot LDS ring per wavefront */
  VPQ_QMV_ROWS = 6,        /* M <= 2, any K % 64: a wavefront streams whole rows with full-width loads, packed bf16
                              dot products, no LDS; what AUTO takes for M <= 2 where K is not a multiple of 512 */
  VPQ_QMV_FLOW = 7,        /* M = 1, K % 512 == 0, K >= 2048: one wavefront per (row set, K part), every load of the
                              launch requested up front, x in registers, scales / biases staged in LDS; what AUTO
                              takes for M = 1 below lm_head-sized packs */
  VPQ_QMV_RING_SPLITK = 8  /* as 5 with K split across workgroups (up to 4 parts, K >= 1024): fp32 planes in `ws`, added
                              in part order by a fold launch that rounds once -- the deep-K split of
                              generative-models/shared/mma-splitk.h:30-52.  AUTO takes it by itself for 2..16 rows when
                              `ws` is given and its cost model says it pays (many rows of x, deep K, narrow N) */
};

/* ---- a6/a7/a8 (+a10): QMM ----------------------------------------------
 * Replaces `affine_qmm_steel_w4g64[_bm64|_bm128]`
 * (gpu-kernels/metal/quant/affine_qmm_steel.metal:461-561; slots 0:w 1:scales
 * 2:biases 3:x 4:y 5:K 6:N 7:M), `affine_qmm_mma_w4g64`
 * (affine_qmm_mma.metal:50-128) and the dequant-once route
 * (generative-models/minimax-h3/metal-minimax-h3-transformer.cc:2020-2160):
 * y[M,N] = bf16_rne( x[M,K] . bf16(W)^T ) -- the weight tile is dequantized in
 * fp32 and rounded to bf16 once (affine_qmm_steel.metal:78-96), contracted on
 * bf16 MFMA with fp32 accumulation, one rounding on store.  M and N need not be
 * tile multiples (affine_qmm_steel.metal:304-317).
 * With a LoRA (lora_a [r,K], lora_b [N,r], bf16, checkpoint orientation --
 * generative-models/lora-fusion.h:20-27): t = bf16(alpha * bf16(x . A^T)) is
 * written to lora_t_ws [M,r] first (the SCALED tile,
 * gpu-kernels/metal/gemm/dense_gemm_mma.metal:227-273), then t . B^T is added
 * into the same fp32 accumulator before the single store (the fused tile,
 * dense_gemm_mma.metal:297-348).  lora_a == NULL or alpha == 0 means no adapter,
 * and the output is then bit-identical to the call without one
 * (metal-minimax-h3-transformer.cc:2211-2219).
 * Requires K % 64 == 0, M, N > 0, and with a LoRA r % 8 == 0, 8 <= r <= VPQ_LORA_MAX_RANK (the reference's
 * LoraFactors.rank is unconstrained, metal-minimax-h3-transformer.h:923-931; it runs rank 16 adapters, .h:365-367,
 * and measures rank 384, .cc:1126-1132); x, y rows may be of any length (K, N) but the base pointers must be
 * 16-byte aligned. */
int vpq_qmm_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* x, uint16_t* y,
                       int K, int N, int M,
                       const uint16_t* lora_a, const uint16_t* lora_b, int r, float alpha,
                       uint16_t* lora_t_ws);

/* The same with the kernel named: tile_n = 128 is the 256 x 128 tile kernel (any K % 64 == 0),
 * 192 / 256 / -128 the large-tile kernel at width 192 / 256 / 128 (needs K % 512 == 0 and 16-byte
 * aligned scales and biases, else VPQ_ERR_BAD_SHAPE), which vpq_qmm_w4g64_bf16 takes by itself once
 * its tiles fill the CUs (the prefill and video-DiT projections), at the width a small cost model
 * picks.  Both kernels accumulate K in the same order with the same instruction: their
 * results are bit-identical.  For measurement and tests; no counterpart in the reference. */
int vpq_qmm_tiled_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                             const uint16_t* lora_a, const uint16_t* lora_b, int r, float alpha,
                             uint16_t* lora_t_ws, int tile_n);

/* Split-K form of the fused kernel for GEMMs with few output tiles (M of a few
 * hundred rows, or a narrow N, over a long K), where one workgroup per 256 x 128
 * tile leaves most of the chip idle and each walks a long serial K loop: `splits`
 * (2..16; 0 = chosen so that about one workgroup per CU results, at least 512 of K
 * each; 1 = none) shares of K run as separate workgroups into fp32 planes
 * [splits][M][N] in `ws`, and a fold adds the planes in order and rounds once.  The
 * model is the reference's deep-K split (generative-models/shared/mma-splitk.h:
 * 30-52, 66-140: f32 planes + fold, chosen by chunk width); results differ from the
 * unsplit kernel only by the fp32 reassociation and are bit-reproducible.  No
 * adapter, no gated store.  `ws`: vpq_qmm_workspace_bytes() bytes (0 where the
 * automatic choice is not to split), 256-byte aligned, contents irrelevant.
 * VPQ_ERR_WORKSPACE if it is needed and missing or too small. */
size_t vpq_qmm_workspace_bytes(int K, int N, int M);
int vpq_qmm_splitk_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const uint16_t* x, uint16_t* y,
                              int K, int N, int M, int splits, void* ws, size_t ws_bytes);

/* ---- a8: the dequant-once route -------------------------------------------
 * Replaces `gemm_mma_` (generative-models/minimax-h3/metal-minimax-h3-transformer.cc:
 * 2020-2160: `affine_dequant_w4g64` into a scratch, then a dense matrix-unit GEMM,
 * gpu-kernels/metal/gemm/dense_gemm_mma.metal:44-93): the pack is expanded into
 * `w_deq` (bf16 [N,K], caller-owned, 2*N*K bytes, 16-byte aligned) and
 * y = bf16( x . w_deq^T ) is computed by the library's own dense GEMM (the
 * large-tile MFMA kernel with the weight tile loaded instead of dequantized:
 * bf16 operands, fp32 accumulation over K in ascending order, one rounding).
 * Same arithmetic as vpq_qmm_w4g64_bf16.  `expand` != 0 runs the expansion
 * first; 0 says that `w_deq` already holds this pack's expansion (a weight is
 * immutable after load, so a caller with the room expands each Linear once).
 * No adapter on this route; nothing is allocated and no other library is
 * loaded.  Requires K % 32 == 0 (K % 64 == 0 for the 64-wide groups of this
 * entry point anyway).  On MI355X this route is the faster one where M is very
 * large (measured at M = 16320: 1.3 PFLOP/s against 1.2 fused) and the fused
 * kernel elsewhere or where the 2*N*K bytes are not available. */
int vpq_qmm_dense_route_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y,
                                   int K, int N, int M, uint16_t* w_deq, int expand);
/* The same route with the runtime adapter of vpq_qmm_w4g64_bf16 (arguments and requirements of both): the pre-pass,
 * the expansion (expand != 0) or the kept one, the dense GEMM with t . B^T in the same accumulators; the result has
 * the bits of vpq_qmm_w4g64_bf16 with that adapter.  Worth it where the tiles are many (M in the thousands). */
int vpq_qmm_dense_route_lora_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                        const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                        uint16_t* w_deq, int expand, const uint16_t* lora_a, const uint16_t* lora_b,
                                        int r, float alpha, uint16_t* lora_t_ws);

/* The adapter's first GEMM alone: t[M,r] = bf16(alpha * bf16(x . A^T)), r % 8 == 0, 8 <= r <= VPQ_LORA_MAX_RANK.
 * Replaces `lora_gemm_a_` (metal-minimax-h3-transformer.cc:1030-1067). */
#define VPQ_LORA_MAX_RANK 512
int vpq_lora_a_bf16(vpq_stream_t stream, const uint16_t* x, const uint16_t* lora_a, uint16_t* t,
                    int M, int K, int r, float alpha);

/* ---- a5: the size-based entrance ----------------------------------------
 * Replaces `MetalQwenModel::qmm_auto_`
 * (generative-models/qwen3/metal-qwen-model.cc:3964-4033) with its ladder
 * (:3839-3962: GEMV, a batched plan that walks M in slabs, the tiled GEMM): up
 * to 64 rows run the QMV arithmetic in slabs of at most 16 rows (one launch per
 * slab), larger M the QMM arithmetic.  (The reference crosses over to the GEMM at
 * M = 8; here the 256-row GEMM tile does not pay below ~64 rows: measured 57 us at
 * 4096->4096 for any M <= 256 against ~10 us per slab.)  Above 32 rows the GEMM
 * splits K (vpq_qmm_splitk_w4g64_bf16) where that pays and `ws` has
 * vpq_qmm_workspace_bytes() bytes (without that room, 33..64 rows stay slabs).  From 8192 rows on, when `ws` holds the
 * expanded weight (N*K*2 bytes), the GEMM runs by the dequant-once route
 * (vpq_qmm_dense_route_w4g64_bf16: expansion + dense GEMM, the reference's route
 * for large M, minimax-h3/metal-minimax-h3-transformer.cc:2020-2160), which is the
 * faster one there; below that, or without that room, the fused kernels.
 * vpq_linear_workspace_bytes() is the size that lets the entrance take its best
 * route for the shape (0: none needed); `ws` is 256-byte aligned scratch whose
 * contents are irrelevant and undefined afterwards. */
size_t vpq_linear_workspace_bytes(int K, int N, int M);
int vpq_linear_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                          const uint16_t* biases, const uint16_t* x, uint16_t* y,
                          int K, int N, int M, void* ws, size_t ws_bytes);

/* ---- several projections of one x in one launch ------------------------
 * Replaces `affine_qmv_qkv_w4g64` (gpu-kernels/metal/quant/affine_qmv.metal:
 * 405-516; slots 0:w 1:scales 2:biases 3:x 4:q_out 5:k_out 6:v_out 7:K
 * 8:q_rows 9:k_rows 10:v_rows), the reference's answer to separate small
 * GEMVs that under-occupy the GPU: `count` (1..4) packs [N_i, K] that share
 * x [M,K], K and M are contracted by ONE kernel launch, each into its own
 * y_i [M,N_i].  The row-concatenated q|k|v weight of the reference is the
 * case w[1] = w[0] + q_rows*K/8 words (scales, biases alike); gate|up of an
 * MLP is count = 2.  Arithmetic and requirements are those of
 * vpq_qmv_w4g64_bf16 per pack (no residual); results are bit-identical to
 * `count` separate calls of its VPQ_QMV_FLOW kernel at M = 1 (K % 512 == 0,
 * K >= 2048), of its VPQ_QMV_MFMA kernel at other M where K % 512 == 0, of
 * its VPQ_QMV_ROWS kernel for other K at M <= 2.  The pointer tables are
 * host arrays, read before the call returns.  Shapes neither grouped kernel
 * takes (K % 512 != 0 with M > 2) run as separate launches. */
int vpq_qmv_group_w4g64_bf16(vpq_stream_t stream, int count, const uint32_t* const* w,
                             const uint16_t* const* scales, const uint16_t* const* biases,
                             const uint16_t* x, uint16_t* const* y, int K, const int* N, int M);

/* ---- fused gate|up projection + SwiGLU -----------------------------------
 * The MLP of every LM family stores gate and up as ONE pack [N = 2*ffn, K] with
 * the rows interleaved by output feature (row 2g = gate row g, row 2g+1 = up
 * row g), built once at load
 * (generative-models/llama3/metal-llama-model.cc:151-188), so that the
 * activation fuses into the store and y is the HALVED [M, ffn]:
 *     y[m, g] = bf16( silu(gate) * up ),  silu(v) = v / (1 + exp(-v)),
 * evaluated in fp32 on the un-rounded sums, one rounding.
 *
 * vpq_interleave_rows builds the interleaved arrays on the device: out row 2i =
 * a row i, out row 2i+1 = b row i, `rows` rows of `row_bytes` (even) bytes each;
 * call it for the codes (row_bytes = K/2), the scales and the biases (K/32). */
int vpq_interleave_rows(vpq_stream_t stream, const void* a, const void* b, void* out,
                        size_t row_bytes, size_t rows);

/* Replaces `affine_qmv_swiglu_w4g64` (gpu-kernels/metal/quant/affine_qmv.metal:
 * 816-906; slots 0:w 1:scales 2:biases 3:x 4:y[M,N/2] 5:K 6:N=2*ffn), QMV
 * arithmetic, 1 <= M <= 16, N even.  `variant` as in vpq_qmv_w4g64_bf16
 * (VPQ_QMV_STREAM has no such epilogue). */
int vpq_qmv_swiglu_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const uint16_t* x, uint16_t* y,
                              int K, int N, int M, int variant);

/* Same, fp32 [M,N/2] output before the final rounding (measurement). */
int vpq_qmv_swiglu_w4g64_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, const uint16_t* x, float* y,
                                int K, int N, int M, int variant);

/* Replaces `affine_qmm_swiglu_w4g64` and its strided twin
 * (gpu-kernels/metal/quant/affine_qmm_steel.metal:663-768: qmm_t_swiglu_rs_impl;
 * slots 0:w 1:scales 2:biases 3:x 4:y 5:K 6:N=2*ffn 7:M [8:out_stride 9:out_off]),
 * QMM arithmetic, any M:  y[m*out_rs + out_off + g] = bf16(silu(gate)*up) with
 * out_rs = out_stride if > 0, else N/2 (then out_off must be 0). */
int vpq_qmm_swiglu_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const uint16_t* x, uint16_t* y,
                              int K, int N, int M, int out_stride, int out_off);

/* The size-based entrance of the fused MLP first half, as the reference's call
 * sites choose between the two (generative-models/llama3/metal-llama-model.cc:
 * 466-477 decode, 634-650 and 800-812 prefill): up to 64 rows the QMV arithmetic
 * in slabs of 16 rows, larger M the QMM arithmetic (as vpq_linear_w4g64_bf16). */
int vpq_linear_swiglu_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                 const uint16_t* biases, const uint16_t* x, uint16_t* y,
                                 int K, int N, int M);

/* The same fused stores with the activation chosen by the caller: VPQ_GATE_SWIGLU
 * as above, VPQ_GATE_GEGLU = gelu_tanh(gate) * up with
 * gelu_tanh(g) = 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))), which replaces
 * `affine_qmv_geglu_w4g64` (gpu-kernels/metal/quant/affine_qmv.metal:1352-1447)
 * and `affine_qmm_geglu_w4g64` (affine_qmm_steel.metal:1460-1572); pack layout,
 * shapes and requirements as for the SwiGLU entries, which are these with
 * activation = VPQ_GATE_SWIGLU. */
enum { VPQ_GATE_SWIGLU = 1, VPQ_GATE_GEGLU = 2 };
int vpq_qmv_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y,
                             int K, int N, int M, int variant, int activation);
/* `affine_qmv_gelu_mul_w4g64` (affine_qmv.metal:751-768, the store :268-279): the per-layer-input gate GEMV,
 * y[n] = bf16(gelu_tanh(v) * mul[n]) with v the GEMV's result already rounded to bf16 (so the output equals the
 * unfused GEMV + activation that reads y back); one row of x, mul bf16 [N].  Requirements of vpq_qmv_w4g64_bf16. */
int vpq_qmv_gelu_mul_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                const uint16_t* mul);
int vpq_qmv_gated_w4g64_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                               const uint16_t* biases, const uint16_t* x, float* y,
                               int K, int N, int M, int variant, int activation);
int vpq_qmm_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y,
                             int K, int N, int M, int out_stride, int out_off, int activation);
int vpq_linear_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, const uint16_t* x, uint16_t* y,
                                int K, int N, int M, int activation);

/* ---- MoE: gathered expert projections (decode and pair-batched prefill) ----
 * The router picks top_k of n_experts experts per token: npair = M*top_k
 * (token, expert) pairs in the order token*top_k + slot, pair_eid[p] (device,
 * int32) the expert of pair p.  An expert tensor is a BATCH of packs
 * [n_experts, N, K/8] (scales, biases [n_experts, N, K/64]); one launch runs
 * the QMV of every pair against its expert's slab
 * (generative-models/qwen3/metal-qwen-model.cc:4190-4206).
 *
 * vpq_gather_qmv_gated_w4g64_bf16 replaces `affine_gather_qmv_swiglu_w4g64`
 * (gpu-kernels/metal/quant/affine_qmv.metal:928-960; slots 0:w 1:scales
 * 2:biases 3:x[M,K] 4:y[npair,N/2] 5:K 6:N=2*inner 7:pair_eid 8:top_k) and
 * `affine_gather_qmv_geglu_w4g64` (:1494-1522): pair p contracts the
 * interleaved gate|up slab of expert pair_eid[p] with x row p / top_k and
 * stores act(gate)*up into y row p.
 * vpq_gather_down_qmv_w4g64_bf16 replaces `affine_gather_down_qmv_w4g64`
 * (:1265-1292; slots 0..6 the same with x[npair,K], y[npair,N], 7:pair_eid):
 * pair p contracts the down slab with x row p into y row p, un-weighted (the
 * routing weight is applied by the combine that follows).
 * QMV arithmetic; a pair's result is bit-identical to the plain call
 * (VPQ_QMV_ROWS) on that expert's slab and that row of x.  A pair whose id is
 * outside [0, n_experts) gets zeros (the reference reads out of bounds there).
 * Requires K % 64 == 0, 1 <= npair <= 65535, top_k >= 1, N even for the gated
 * form; w, x 16-byte aligned. */
int vpq_gather_qmv_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                    const int32_t* pair_eid, int npair, int top_k, int n_experts, int activation);
int vpq_gather_down_qmv_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                   const int32_t* pair_eid, int npair, int n_experts);

/* ---- MoE: expert-sorted GEMV, two slots per tile ---------------------------
 * For a few rows per expert the reference sorts the (token, expert) pairs
 * into per-expert tiles of MAXM = 2 slots and runs a GEMV that reads the
 * expert's slab once per tile instead of once per pair
 * (gpu-kernels/metal/quant/affine_qmv.metal:2551-2719).  vpq_moe_sort_pairs
 * with block_rows = VPQ_QMV_GROUPED_SLOTS builds tile2e / srow for it.
 *
 * vpq_qmv_grouped_gated_w4g64_bf16 replaces `affine_grouped_swiglu_w4g64`
 * (:2707; slots 0:w 1:scales 2:biases 3:x[rows,K] 4:y[npad,N/2] 5:K 6:N
 * 7:srow 8:tile2e; grid.z = tile): slot s of tile t reads x row srow[s] and
 * stores act(gate)*up of expert tile2e[t]'s interleaved gate|up slab into y
 * row s.  vpq_qmv_grouped_down_w4g64_bf16 replaces `affine_grouped_down_w4g64`
 * (:2708): x[npad,K] and y[npad,N] both in slot order.  A slot with
 * srow[s] < 0 is padding and a tile with tile2e[t] < 0 (or an id >=
 * n_experts) is unused: nothing is written for them.  A live slot's result is
 * bit-identical to the plain call (VPQ_QMV_ROWS) on that slab and that row.
 * Requires K % 64 == 0, npad a positive multiple of VPQ_QMV_GROUPED_SLOTS,
 * npad / 2 <= 65535, N even for the gated form; w, x 16-byte aligned. */
#define VPQ_QMV_GROUPED_SLOTS 2
int vpq_qmv_grouped_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int npad,
                                     const int32_t* tile2e, const int32_t* srow, int n_experts, int activation);
int vpq_qmv_grouped_down_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int npad,
                                    const int32_t* tile2e, const int32_t* srow, int n_experts);
/* Rows of the sorted down projection back to pair order: replaces `moe_scatter_back_f16`
 * (gpu-kernels/metal/ops/llm_elementwise.metal:328-342; slots 0:dsorted[npad,H] 1:sdst[npad] 2:partials[npair,H] 3:H):
 * partials[sdst[s], :] = dsorted[s, :] for every slot with 0 <= sdst[s] < npair (padding slots are skipped; the
 * reference does not check the upper bound).  A copy of 2-byte elements: serves both element types. */
int vpq_moe_scatter_back_bf16(vpq_stream_t stream, const uint16_t* dsorted, const int32_t* sdst,
                              uint16_t* partials, int npad, int H, int npair);
/* The same over a batched 8-bit pack [E, N, K/4]: `affine_grouped_swiglu_w8g64`, `affine_grouped_down_w8g64`
 * (affine_qmv.metal:2718-2719).  A live slot is bit-identical to the pair-gathered 8-bit call
 * (vpq_gather_qmv_gated_w8g64_bf16 / vpq_gather_down_qmv_w8g64_bf16) of that expert on that row. */
int vpq_qmv_grouped_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int npad,
                                     const int32_t* tile2e, const int32_t* srow, int n_experts, int activation);
int vpq_qmv_grouped_down_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int npad,
                                    const int32_t* tile2e, const int32_t* srow, int n_experts);

/* ---- MoE prefill: expert-sorted (grouped) GEMMs ---------------------------
 * With many tokens the pairs are sorted by expert into blocks of
 * vpq_qmm_grouped_block_rows() slots, each block owned by ONE expert, and two
 * tiled GEMMs run over the sorted slots, reading every expert slab once per
 * block instead of once per pair
 * (generative-models/qwen3/metal-qwen-model.cc:4209-4264).
 *
 * vpq_moe_sort_pairs replaces the sort's four dispatches `moe_ifill_i32`,
 * `moe_hist_i32`, `moe_sort_setup_i32`, `moe_scatter_i32`
 * (gpu-kernels/metal/ops/llm_elementwise.metal:255-326) with the reference's
 * sizing: max_tiles >= ceil(npair / block_rows) + min(n_experts, npair) blocks,
 * npad = max_tiles * block_rows slots.  Outputs (device, int32):
 * tile2e[max_tiles] expert per block (-1 unused), srow[npad] token row per slot
 * (= pair / top_k; -1 padding), sdst[npad] pair per slot (-1 padding),
 * ntiles[1] blocks in use.  Experts ascend; the order of the pairs inside an
 * expert's share is unspecified, as in the reference.  A pair whose id is
 * outside [0, n_experts) gets no slot.  ws: vpq_moe_sort_workspace_bytes()
 * bytes of device memory, 4-byte aligned.  block_rows is any positive count
 * (the GEMMs below need vpq_qmm_grouped_block_rows()).
 *
 * vpq_qmm_grouped_gated_w4g64_bf16 replaces `affine_qmm_grouped_swiglu_w4g64`
 * and `affine_qmm_grouped_geglu_w4g64` (gpu-kernels/metal/quant/
 * affine_qmm_steel.metal:1314-1339, 1266-1288; slots 0:w[E,N,K/8] 1:scales
 * 2:biases 3:x[rows_x,K] 4:y[npad,N/2] 5:K 6:N=2*inner 7:npad 8:tile2e 9:srow):
 * slot i contracts x row srow[i] with the interleaved gate|up slab of its
 * block's expert and stores act(gate)*up into y row i; a padding slot
 * (srow < 0, or >= rows_x) stores zeros, as the reference's zero-filled rows do;
 * a block with tile2e < 0 (or >= n_experts) is left untouched.
 * vpq_qmm_grouped_down_w4g64_bf16 replaces `affine_qmm_grouped_w4g64`
 * (:1042-1066; 3:x[npad,K] sorted activations 4:y[rows_y,N] 9:sdst): slot i
 * contracts x row i with the down slab and stores into y row sdst[i]
 * (nothing for sdst < 0 or >= rows_y).
 * QMM arithmetic (bf16-rounded weight, fp32 accumulation over K ascending, one
 * rounding): a slot's result has the bits of vpq_qmm_tiled_w4g64_bf16 (tile
 * 128) on that row and that expert's slab.  Requires K % 64 == 0, npad a
 * positive multiple of vpq_qmm_grouped_block_rows(), N even for the gated form,
 * rows * K * 2 < 4e9 for x; w, x 16-byte aligned, y 8-byte aligned (its rows are
 * stored in 4- and 8-byte pieces). */
int vpq_qmm_grouped_block_rows(void);
size_t vpq_moe_sort_workspace_bytes(int n_experts);
int vpq_moe_sort_pairs(vpq_stream_t stream, const int32_t* pair_eid, int npair, int top_k, int n_experts,
                       int block_rows, int max_tiles, int32_t* tile2e, int32_t* srow, int32_t* sdst,
                       int32_t* ntiles, void* ws, size_t ws_bytes);
int vpq_qmm_grouped_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                     int npad, const int32_t* tile2e, const int32_t* srow, int n_experts,
                                     int rows_x, int activation);
int vpq_qmm_grouped_down_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                    int npad, const int32_t* tile2e, const int32_t* sdst, int n_experts,
                                    int rows_y);

/* ---- 4-bit group-32 twins (w4g32; GGUF Q4_0 repacked to affine) ---------------
 * The 4-bit pack with a scale and a bias per 32 values: w uint32 [N, K/8] as
 * above, scales, biases bf16 [N, K/32].
 *   vpq_dequant_w4g32_bf16           replaces `affine_dequant_w4g32`
 *                                    (gpu-kernels/metal/quant/affine_dequant.metal:196-228), bit-exact.
 *   vpq_qmv_w4g32_bf16 / _f32out     replace `affine_qmv_w4g32[_add]` (affine_qmv.metal:305-320,
 *                                    367-384) and, with scale_only != 0, the Q4_0 forms
 *                                    `affine_qmv_w4g32[_add]_q40` (:327-342, 387-403): the bias is
 *                                    -8 * scale computed in registers and `biases` is never read
 *                                    (may be NULL) -- bit-identical to the affine form on a pack
 *                                    whose stored bias is -8 * scale, 10 % fewer bytes.
 *                                    QMV arithmetic, 1 <= M <= 16.
 *   vpq_qmv_gated_w4g32_bf16         replaces `affine_qmv_geglu_w4g32[_q40]` (:1451-1490) and the
 *                                    SwiGLU twin over an interleaved gate|up pack; y [M, N/2].
 *   vpq_qmm_w4g32_bf16, vpq_qmm_gated_w4g32_bf16   the fused kernels with a scale and a bias per 32
 *                                    values: replace `affine_qmm_steel_w4g32`
 *                                    (affine_qmm_steel.metal:618-640) and `affine_qmm_geglu_w4g32`
 *                                    (:1573-1596) plus the SwiGLU twin; K % 64 == 0, any M.  Chosen by size as
 *                                    for the group-64 pack: the large-tile kernel once its tiles fill the CUs
 *                                    (K % 512 == 0, 16-byte aligned scales / biases), else the 256 x 128 tile
 *                                    kernel; the two give the same bits.
 *   vpq_qmm_dense_route_w4g32_bf16   GEMM by expansion into w_deq[N,K] + the library's dense GEMM
 *                                    (expand as in vpq_qmm_dense_route_w4g64_bf16).
 * Requires K % 32 == 0; w, x 16-byte aligned. */
int vpq_dequant_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, uint16_t* w_deq, int K, int N);
int vpq_qmv_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       const uint16_t* x, uint16_t* y, int K, int N, int M, const uint16_t* residual,
                       int scale_only);
int vpq_qmv_w4g32_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                         const uint16_t* x, float* y, int K, int N, int M, int scale_only);
int vpq_qmv_gated_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, uint16_t* y, int K, int N, int M, int activation, int scale_only);
int vpq_qmm_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       const uint16_t* x, uint16_t* y, int K, int N, int M);
/* As vpq_qmm_tiled_w8g64_bf16 for the group-32 pack (tile_n 128, -128, 256; the large-tile kernel has no 192-wide
 * form for groups of 32: VPQ_ERR_BAD_SHAPE). */
int vpq_qmm_tiled_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y,
                             int K, int N, int M, int activation, int tile_n);
/* The size-based entrance over a group-32 pack: slabs of vpq_qmv_w4g32_bf16 up to 64 rows (at every M where
 * K % 64 != 0), vpq_qmm_w4g32_bf16 above. */
int vpq_linear_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                          const uint16_t* x, uint16_t* y, int K, int N, int M);
int vpq_qmm_gated_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, uint16_t* y, int K, int N, int M, int activation);
int vpq_qmm_dense_route_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                   uint16_t* w_deq, int expand);

/* ---- greedy tail: argmax of the lm_head's logits on the device ------------------
 * Replaces `argmax_f16` (gpu-kernels/metal/ops/llm_elementwise.metal:2906-2941;
 * slots 0:logits 1:out_id 2:V), and the two-stage pair `argmax_partial_f16`
 * (:2977-3028; 0:logits 1:partials 2:V 3:M) + `argmax_combine_f16` (:3030-3062;
 * 0:partials 1:out_id 2:M), which keep the sampled token on the device: out_id
 * is read back by the next step's embedding gather as its `ids`.
 * out_id[r] = index of the largest of the V bf16 logits of row r, the LOWEST
 * index among equal maxima (a left-to-right `v > best` scan), a NaN never
 * wins; 0 for a row of nothing but NaNs.  Exact, whatever the reduction order.
 *   vpq_argmax_bf16          logits [rows, V] -> out_id [rows].  With ws == NULL one
 *                            workgroup scans a row; with vpq_argmax_workspace_bytes(V, rows)
 *                            bytes of ws (4-byte aligned) a row is scanned by slabs and combined.
 *   vpq_argmax_partial_bf16  one row: `parts` (1..65535) contiguous slabs -> partials, 2*parts
 *                            4-byte slots (value as fp32, index as int32; opaque to the caller).
 *   vpq_argmax_combine       partials of one row -> out_id[0]. */
size_t vpq_argmax_workspace_bytes(int V, int rows);
int vpq_argmax_bf16(vpq_stream_t stream, const uint16_t* logits, int32_t* out_id, int V, int rows,
                    void* ws, size_t ws_bytes);
int vpq_argmax_partial_bf16(vpq_stream_t stream, const uint16_t* logits, float* partials, int V, int parts);
/* The two-stage vpq_argmax_bf16 for callers that cannot allocate or pass a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The slab
 * pairs go to a static device array of the library (128 KB per GPU, held until the process ends) instead of
 * `ws`; the call allocates nothing and gives the bits of vpq_argmax_bf16 with a workspace.  rows is limited to
 * VPQ_ARGMAX_STATIC_MAX_ROWS (more: VPQ_ERR_WORKSPACE, with the limit in vpq_last_device_error()); V is not.
 * All calls on one GPU share the array: calls that overlap on a GPU (two streams, two threads) race; calls in
 * stream order on one stream do not.  vpq_init() resolves the array's address for the current device; else the
 * first call on a device does. */
#define VPQ_ARGMAX_STATIC_MAX_ROWS 64
int vpq_argmax_bf16_static(vpq_stream_t stream, const uint16_t* logits, int32_t* out_id, int V, int rows);
int vpq_argmax_combine(vpq_stream_t stream, const float* partials, int32_t* out_id, int parts);

/* ---- 8-bit group-64 twins (w8g64) -------------------------------------------
 * The same affine format with one BYTE per value: w uint32 [N, K/4],
 * q[n, 4j+i] = (w[n,j] >> 8i) & 0xFF; scales, biases bf16 [N, K/64]
 * (gpu-kernels/metal/quant/affine_dequant.metal:60-97).  A first, general path for
 * the 8-bit checkpoints and the 8-bit linears of mixed-precision ones; not tuned
 * like the 4-bit kernels:
 *   vpq_dequant_w8g64_bf16           replaces `affine_dequant_w8g64` (:68-97), bit-exact.
 *   vpq_qmv_w8g64_bf16 / _f32out     replace `affine_qmv_w8g64[_add]`
 *                                    (affine_qmv.metal:3034-3050, 3122-3140): QMV arithmetic,
 *                                    1 <= M <= 16, one wavefront per output row.
 *   vpq_qmm_dense_route_w8g64_bf16   the dequant-once route for any M (replaces
 *                                    `affine_qmm_steel_w8g64`, affine_qmm_steel.metal:1601-1672,
 *                                    by the reference's own second route): expansion into
 *                                    `w_deq` [N,K] bf16 + the library's dense GEMM; arguments as
 *                                    vpq_qmm_dense_route_w4g64_bf16.
 *   vpq_qmv_gated_w8g64_bf16         replaces `affine_qmv_swiglu_w8g64` and `affine_qmv_geglu_w8g64`
 *                                    (affine_qmv.metal:3140-3178): interleaved gate|up pack
 *                                    [N = 2*ffn, K/4], y [M, N/2] = act(gate) * up, 1 <= M <= 16.
 *   vpq_gather_qmv_gated_w8g64_bf16  replaces `affine_gather_qmv_swiglu_w8g64` (:962-990) and
 *                                    `affine_gather_qmv_geglu_w8g64` (:1524-1552);
 *   vpq_gather_down_qmv_w8g64_bf16   replaces `affine_gather_down_qmv_w8g64` (:1295-1322): the MoE
 *                                    gathers over a batched 8-bit pack [E, N, K/4], arguments and
 *                                    conventions of the 4-bit vpq_gather_* entries; a pair is
 *                                    bit-identical to the plain 8-bit call on that expert's slab.
 *   vpq_qmm_w8g64_bf16, vpq_qmm_gated_w8g64_bf16   the fused kernels with byte codes (the large-tile kernel
 *                                    once its tiles fill the CUs, else the 256 x 128 tile kernel; same bits): replace
 *                                    `affine_qmm_steel_w8g64[_bm64|_bm128]` (affine_qmm_steel.metal:1601-1672)
 *                                    and `affine_qmm_swiglu_w8g64*` / `affine_qmm_geglu_w8g64` (:1700-1890);
 *                                    arguments as vpq_qmm_w4g64_bf16 (no adapter) / vpq_qmm_gated_w4g64_bf16.
 *   vpq_qmm_grouped_gated_w8g64_bf16, vpq_qmm_grouped_down_w8g64_bf16   the expert-sorted MoE GEMMs over a
 *                                    batched 8-bit pack: replace `affine_qmm_grouped_swiglu_w8g64`,
 *                                    `affine_qmm_grouped_geglu_w8g64`, `affine_qmm_grouped_w8g64` (:1069-1090,
 *                                    1290-1312, 1341-1366); arguments as the 4-bit vpq_qmm_grouped_* entries.
 *   vpq_gather_qmv_gated_split_bf16  replaces `affine_gather_qmv_swiglu_w4w8g64` and `_w8w4g64`
 *                                    (:1198-1260; slots 0..2 gate pack, 3..5 up pack, 6:x 7:y 8:K
 *                                    9:ffn 10:pair_eid 11:top_k): gate and up as SEPARATE batched
 *                                    packs [E, ffn, ...] of gate_bits / up_bits in {4, 8} each (what a
 *                                    per-tensor quantizer leaves), y [npair, ffn] = act(gate) * up.
 *                                    pair_eid NULL: no experts, npair <= 16 rows of x.
 * Requirements as for the 4-bit entries (K % 64 == 0; 16-byte aligned w, x). */
int vpq_gather_qmv_gated_split_bf16(vpq_stream_t stream, const uint32_t* wg, const uint16_t* sg, const uint16_t* bg,
                                    int gate_bits, const uint32_t* wu, const uint16_t* su, const uint16_t* bu,
                                    int up_bits, const uint16_t* x, uint16_t* y, int K, int ffn,
                                    const int32_t* pair_eid, int npair, int top_k, int n_experts, int activation);
int vpq_qmm_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M);
/* Names the kernel of the fused 8-bit GEMM (measurement and tests), as vpq_qmm_tiled_w4g64_bf16 does for the
 * 4-bit pack: tile_n 128 = the 256 x 128 tile kernel, 192 = the large-tile kernel (K % 512 == 0, 16-byte
 * aligned scales / biases; byte codes take weight tiles of up to 192 rows), -128 = the large-tile kernel at
 * width 128.  activation 0 = plain y [M,N], else the gated store y [M,N/2].  VPQ_ERR_BAD_SHAPE where the
 * named kernel does not take the shape.  vpq_qmm_w8g64_bf16 / vpq_qmm_gated_w8g64_bf16 choose by size: the
 * large-tile kernel once its tiles fill the CUs. */
int vpq_qmm_tiled_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y,
                             int K, int N, int M, int activation, int tile_n);
/* The size-based entrance over an 8-bit pack (qmm_auto_'s ladder, generative-models/qwen3/
 * metal-qwen-model.cc:3964-4033, which takes the width from the layer): slabs of vpq_qmv_w8g64_bf16 up to
 * 64 rows, vpq_qmm_w8g64_bf16 above. */
int vpq_linear_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                          const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M);
/* `affine_requant_w8_to_w4_g64` (affine_dequant.metal:134-186): the half-width copy of an 8-bit pack (the draft
 * lm_head of speculative decoding).  Per group of 64: v = s8 q8 + b8 in fp32, scale = (max - min) / 15, bias = min,
 * q4 = round-half-away((v - min) / scale) clamped to 0..15 (a constant group: scale 0, codes 0); s4 / b4 are the bf16
 * roundings, the codes use the unrounded fp32 scale.  w8 uint32 [N, K/4], s8 / b8 bf16 [N, K/64] in; w4 uint32
 * [N, K/8], s4 / b4 bf16 [N, K/64] out; K % 64 == 0, w8 and w4 16-byte aligned.  Bit-exact with IEEE division. */
int vpq_requant_w8_to_w4_g64_bf16(vpq_stream_t stream, const uint32_t* w8, const uint16_t* s8, const uint16_t* b8,
                                  uint32_t* w4, uint16_t* s4, uint16_t* b4, int K, int N);
/* The 8-bit and group-32 twins of vpq_qmv_gelu_mul_w4g64_bf16: `affine_qmv_gelu_mul_w8g64` (affine_qmv.metal:788-805)
 * and `affine_qmv_gelu_mul_w4g32` (:769-786; scale_only as in vpq_qmv_w4g32_bf16). */
int vpq_qmv_gelu_mul_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                const uint16_t* mul);
int vpq_qmv_gelu_mul_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                const uint16_t* mul, int scale_only);
/* 8-bit codes in groups of 32 (GGUF q8 repacked to affine; the codec's int8 path): w uint32 [N, K/4], scales / biases
 * bf16 [N, K/32], K % 32 == 0.  vpq_dequant_w8g32_bf16 replaces `affine_dequant_w8g32` (affine_dequant.metal:99-131),
 * bit-exact; vpq_qmv_w8g32_bf16 replaces `affine_qmv_w8g32` (affine_qmv.metal:3053-3069), QMV arithmetic, 1 <= M <= 16;
 * vpq_qmm_dense_route_w8g32_bf16 serves `affine_qmm_steel_w8g32` (affine_qmm_steel.metal:1674-1698) by the
 * dequant-once route the reference's codec itself takes (arguments as vpq_qmm_dense_route_w4g64_bf16). */
int vpq_dequant_w8g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, uint16_t* w_deq, int K, int N);
int vpq_qmv_w8g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                       const uint16_t* residual);
int vpq_qmm_dense_route_w8g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                   uint16_t* w_deq, int expand);
/* `affine_moe_gate_w8g64` (affine_qmv.metal:1323-1349): the shared-expert gate, gate[m] = bf16(sigmoid(W[1,K] . x[m]))
 * for M rows of x (1 <= M <= 65535) over a one-row 8-bit pack (w uint32 [K/4], scales / biases bf16 [K/64]). */
int vpq_moe_gate_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                            const uint16_t* biases, const uint16_t* x, uint16_t* gate, int K, int M);
int vpq_qmm_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                             int out_stride, int out_off, int activation);
int vpq_qmm_grouped_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                     int npad, const int32_t* tile2e, const int32_t* srow, int n_experts,
                                     int rows_x, int activation);
int vpq_qmm_grouped_down_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                    int npad, const int32_t* tile2e, const int32_t* sdst, int n_experts,
                                    int rows_y);
int vpq_qmv_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                             int activation);
int vpq_gather_qmv_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                    const int32_t* pair_eid, int npair, int top_k, int n_experts, int activation);
int vpq_gather_down_qmv_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                   const int32_t* pair_eid, int npair, int n_experts);
int vpq_dequant_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, uint16_t* w_deq, int K, int N);
int vpq_qmv_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* x, uint16_t* y,
                       int K, int N, int M, const uint16_t* residual);
int vpq_qmv_w8g64_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                         const uint16_t* biases, const uint16_t* x, float* y, int K, int N, int M);
int vpq_qmm_dense_route_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y,
                                   int K, int N, int M, uint16_t* w_deq, int expand);

/* ---- IEEE binary16 element type (f16) ------------------------------------
 * The reference builds every kernel for two element types (VPIPE_ELT = bfloat
 * and half: apple-silicon/metal-compute/CMakeLists.txt:71-72, 159-162; the
 * metallibs without the `_bf16` suffix).  These entries are the f16 forms of
 * the 4-bit group-64 functions: scales, biases, x, y, residual and w_deq are
 * IEEE binary16 bit patterns, the packed codes are the same.  One row of x on
 * K % 512 == 0, K >= 2048 with 16-byte aligned scales and biases takes the
 * streaming decode kernel of the bf16 entry on binary16 arithmetic (same
 * speed), 2..16 rows on K % 512 == 0 the ring kernel (VPQ_QMV_RING) or, for 2..4
 * rows over 150 MB of codes and more, the streaming kernel (VPQ_QMV_STREAM) on
 * binary16 arithmetic; every other QMV shape takes a general path (one wavefront per
 * output row); the QMM is expansion + the dense GEMM:
 *   vpq_dequant_w4g64_f16         `affine_dequant_w4g64` (affine_dequant.metal:25-58), bit-exact:
 *                                 f16_rne(fp32(s) * q + fp32(b)).
 *   vpq_qmv_w4g64_f16 / _f32out   `affine_qmv_w4g64[_add]` (affine_qmv.metal:286-301, 347-363),
 *                                 1 <= M <= 16, fp32 accumulation, un-rounded weights.
 *   vpq_qmv_gated_w4g64_f16       `affine_qmv_swiglu_w4g64`, `affine_qmv_geglu_w4g64` (:891-906, 1432-1447).
 *   vpq_qmm_dense_route_w4g64_f16 the dequant-once route (expansion into w_deq [N,K] f16 + the dense
 *                                 GEMM), arguments as vpq_qmm_dense_route_w4g64_bf16.
 *   vpq_qmm_w4g64_f16             the fused GEMM `affine_qmm_steel_w4g64[_bm64|_bm128]` (affine_qmm_steel.metal:
 *                                 470-560) and, with activation VPQ_GATE_SWIGLU / VPQ_GATE_GEGLU, the gated
 *                                 `affine_qmm_swiglu_w4g64*`, `affine_qmm_geglu_w4g64` (y [M,N/2], N even) on
 *                                 binary16 elements: weight tile = f16_rne(fp32(s*q+b)), f16 MFMA, fp32
 *                                 accumulation, one rounding -- the kernels of the bf16 entry (the large-tile
 *                                 kernel once its tiles fill the CUs, K % 512 == 0 and 16-byte aligned scales /
 *                                 biases; the 256 x 128 tile kernel otherwise, any K % 64 == 0); x and y
 *                                 16-byte aligned.  Its results have the bits of the dequant-once route.
 * Requirements as for the bf16 entries. */
int vpq_dequant_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                          const uint16_t* biases, uint16_t* w_deq, int K, int N);
int vpq_qmv_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                      const uint16_t* biases, const uint16_t* x, uint16_t* y,
                      int K, int N, int M, const uint16_t* residual);
int vpq_qmv_w4g64_f16_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, float* y, int K, int N, int M);
int vpq_qmv_gated_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                            const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                            int activation);
int vpq_qmm_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                      const uint16_t* biases, const uint16_t* x, uint16_t* y,
                      int K, int N, int M, int activation);
/* The runtime adapter on binary16 elements (the half build of `lora_gemm_a_` / the SCALED and the fused tile of
 * gpu-kernels/metal/gemm/dense_gemm_mma.metal:227-273, 297-348, whose element type is VPIPE_ELT, :28-33):
 * vpq_lora_a_f16 is t[M,r] = f16(alpha * f16(x . A^T)); vpq_qmm_lora_w4g64_f16 is vpq_qmm_w4g64_f16 (no
 * activation) with y += t . B^T in the same accumulators before the one rounding.  A [r,K], B [N,r], t scratch
 * [M,r], all binary16; r % 8 == 0, 8 <= r <= VPQ_LORA_MAX_RANK; lora_a == NULL or alpha == 0: no adapter. */
int vpq_lora_a_f16(vpq_stream_t stream, const uint16_t* x, const uint16_t* lora_a, uint16_t* t,
                   int M, int K, int r, float alpha);
int vpq_qmm_lora_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                           const uint16_t* lora_a, const uint16_t* lora_b, int r, float alpha,
                           uint16_t* lora_t_ws);
/* The grouped launch on binary16 elements (`affine_qmv_qkv_w4g64` of the half build, affine_qmv.metal:497-516):
 * arguments and results as vpq_qmv_group_w4g64_bf16 -- bit-identical to `count` calls of vpq_qmv_w4g64_f16; one
 * launch at M = 1 on K % 512 == 0, K >= 2048 with 16-byte aligned scales / biases, separate calls otherwise. */
int vpq_qmv_group_w4g64_f16(vpq_stream_t stream, int count, const uint32_t* const* w,
                            const uint16_t* const* scales, const uint16_t* const* biases,
                            const uint16_t* x, uint16_t* const* y, int K, const int* N, int M);
int vpq_qmm_dense_route_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                  const uint16_t* biases, const uint16_t* x, uint16_t* y,
                                  int K, int N, int M, uint16_t* w_deq, int expand);
/* The grouped launch of the format twins (`affine_qmv_qkv_w4g32`, `affine_qmv_qkv_w8g64`, affine_qmv.metal:518-559):
 * arguments as vpq_qmv_group_w4g64_bf16 (w uint32 [N_i, K/8] with scales / biases [N_i, K/32], resp. w uint32
 * [N_i, K/4] with [N_i, K/64]); bit-identical to `count` calls of vpq_qmv_w4g32_bf16 / vpq_qmv_w8g64_bf16.  Group-32
 * packs at M <= 2 run as one launch; the other cases are separate launches behind one call. */
int vpq_qmv_group_w4g32_bf16(vpq_stream_t stream, int count, const uint32_t* const* w,
                             const uint16_t* const* scales, const uint16_t* const* biases,
                             const uint16_t* x, uint16_t* const* y, int K, const int* N, int M, int scale_only);
int vpq_qmv_group_w8g64_bf16(vpq_stream_t stream, int count, const uint32_t* const* w,
                             const uint16_t* const* scales, const uint16_t* const* biases,
                             const uint16_t* x, uint16_t* const* y, int K, const int* N, int M);
/* `affine_qmv_qkv_rms_w4g64` / `_w4g32` / `_w8g64` (affine_qmv.metal:561-740): RMSNorm of the input row and the
 * fused-QKV GEMV over it.  vpq_rmsnorm_bf16 is the norm alone, out[m,k] = bf16(float(x[m,k]) * inv_m * float(norm_w[k])),
 * inv_m = rsqrt(sum_k x[m,k]^2 / K + eps) in fp32 (:601-616; norm_w holds Gemma's 1 + w already), 1 <= M <= 65535.
 * vpq_qmv_qkv_rms_bf16 runs it on the one row x [K] into `x_norm_ws` (K elements of caller scratch, 16-byte aligned:
 * the reference keeps the normalized row in threadgroup memory) and then the grouped GEMV of `format` (VPQ_FORMAT_*)
 * over that row: two launches, the values of the fused kernel. */
enum { VPQ_FORMAT_W4G64 = 0, VPQ_FORMAT_W4G32 = 1, VPQ_FORMAT_W8G64 = 2, VPQ_FORMAT_W8G32 = 3 };
int vpq_rmsnorm_bf16(vpq_stream_t stream, const uint16_t* x, const uint16_t* norm_w, uint16_t* out,
                     int K, int M, float eps);
int vpq_qmv_qkv_rms_bf16(vpq_stream_t stream, int format, int count, const uint32_t* const* w,
                         const uint16_t* const* scales, const uint16_t* const* biases, const uint16_t* x,
                         const uint16_t* norm_w, uint16_t* const* y, int K, const int* N, float eps,
                         uint16_t* x_norm_ws);
/* 8-bit codes on IEEE binary16 elements -- the half build of `affine_dequant_w8g64` / `affine_dequant_w8g32`
 * (affine_dequant.metal:60-131) and of `affine_qmm_steel_w8g64` / `_w8g32` (affine_qmm_steel.metal:1601-1698), which is
 * what the reference's codec runs (moss/metal-moss-codec.cc:181-183, 579-581): scales, biases, x, y and w_deq are
 * binary16, group is 64 or 32.  The expansion is bit-exact (f16(fp32(s q + b)), the product exact); the GEMM goes by the
 * dequant-once route on the binary16 dense GEMM (arguments of vpq_qmm_dense_route_w4g64_f16). */
int vpq_dequant_w8_f16(vpq_stream_t stream, int group, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, uint16_t* w_deq, int K, int N);
int vpq_qmm_dense_route_w8_f16(vpq_stream_t stream, int group, const uint32_t* w, const uint16_t* scales,
                               const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                               uint16_t* w_deq, int expand);
/* The dequant-once route with the runtime adapter over a pack of any format (VPQ_FORMAT_*: the 4-bit group-64 form is
 * vpq_qmm_dense_route_lora_w4g64_bf16, whose arguments these are): the adapter's pre-pass into lora_t_ws, the format's
 * expansion into w_deq (expand != 0) or the kept one, then the dense GEMM with t . B^T in the same accumulators -- the
 * reference's route for an adapter over a quantized Linear of any width (`gemm_`, metal-minimax-h3-transformer.cc:
 * 2205-2259, with Linear.bits 4 or 8).  The fused kernels of the 8-bit and group-32 packs take no adapter; this is
 * their adapter path.  With an adapter K % 64 == 0. */
int vpq_qmm_dense_route_lora_bf16(vpq_stream_t stream, int format, const uint32_t* w, const uint16_t* scales,
                                  const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                  uint16_t* w_deq, int expand, const uint16_t* lora_a, const uint16_t* lora_b,
                                  int r, float alpha, uint16_t* lora_t_ws);

/* ---- a12: the packer ------------------------------------------------------
 * Replaces `affine_quant_w4_g64` (gpu-kernels/metal/quant/affine_dequant.metal:
 * 243-301; slots 0:x 1:w 2:s 3:b 4:K 5:N 6:clip) driven by
 * AffineQuantizer::quantize_linear (generative-models/quantize/affine-quantizer.cc:
 * 52-84): per 64-wide group scale = (max-min)/15, bias = min,
 * q = clamp(round((v-min)/scale), 0, 15); scales and biases are emitted as IEEE
 * F16 bit patterns, the on-disk format.  `src` is bf16 [N,K]. */
int vpq_quantize_w4g64(vpq_stream_t stream, const uint16_t* src, uint32_t* w,
                       uint16_t* scales_f16, uint16_t* biases_f16, int K, int N, float clip);
/* The same packer for every width and group of the reference (`affine_quant_w4_g64`, `_w4_g32`, `_w8_g64`, `_w8_g32`,
 * affine_dequant.metal:243-301): bits 4 or 8, group 64 or 32, scale = (max - min) / (2^bits - 1); w is
 * [N, K * bits / 32] words, scales / biases F16 [N, K / group]; K % group == 0.  src_f16 != 0: `src` is IEEE binary16
 * (the build the reference's quantizer runs, generative-models/quantize/affine-quantizer.cc:25), else bf16. */
int vpq_quantize(vpq_stream_t stream, int bits, int group, int src_f16, const uint16_t* src, uint32_t* w,
                 uint16_t* scales_f16, uint16_t* biases_f16, int K, int N, float clip);

/* F16 -> bf16 conversion of scales / biases a bf16 model does once at load
 * (docs/PLUGINS.md:210-213). */
int vpq_f16_to_bf16(vpq_stream_t stream, const uint16_t* in_f16, uint16_t* out_bf16, size_t count);

/* ---- the stochastic sampler tail ------------------------------------------
 * vpq_sample_topp_bf16 replaces `sample_topp_f16`
 * (gpu-kernels/metal/ops/llm_elementwise.metal:3116-3262; slots 0:logits
 * 1:out_id 2:V 3:temp 4:top_p 5:seed 6:ws 7:n_iter 8:rep_penalty
 * 9:presence_penalty 10:top_k 11:min_p 12:seen; one threadgroup): the whole
 * sampler over one row of bf16 logits on the device, in the host sampler's
 * order -- repetition and presence penalty on the tokens marked in `seen`
 * ([V] bytes, in/out: the drawn token is marked), temperature, softmax weights
 * (cached in `ws`, [V] bf16 scratch), top-k (0 or >= V: off), min-p, top-p as
 * weight thresholds found by n_iter bisection steps each, then a Gumbel-max
 * draw over the kept set with a hash of (seed, index), lowest index on ties;
 * token 0 if nothing is kept.  The draw is an exact function of its inputs:
 * exp, log and the reduction order are fixed (see vpq_sample.hip), so the
 * same (logits, seen, parameters, seed) give the same token on every run.
 * One workgroup: ~0.5-0.9 ms at 151936 logits; see vpq_sample_hist_bf16.
 * Requires V >= 1, n_iter >= 0, rep != 0; all pointers non-NULL, logits and ws
 * 2-byte, out_id 4-byte aligned. */
int vpq_sample_topp_bf16(vpq_stream_t stream, const uint16_t* logits, int32_t* out_id, int V, float temp,
                         float top_p, uint32_t seed, uint16_t* ws, int n_iter, float rep_penalty,
                         float presence_penalty, int top_k, float min_p, uint8_t* seen);

/* vpq_sample_hist_bf16 replaces the reference's multi-threadgroup sampler
 * `sample_max_partial_f16`, `sample_max_combine_f16`, `sample_zhist_partial_f16`,
 * `sample_zhist_combine_f16`, `sample_thresh_f16`, `sample_pick_partial_f16`,
 * `sample_pick_combine_f16` (llm_elementwise.metal:3255-3640; its M is n_slabs
 * here) -- seven dispatches there, one call (five launches) here.  Same
 * pipeline and arguments as vpq_sample_topp_bf16 without n_iter: the
 * vocabulary is cut into n_slabs contiguous slabs of ceil(V / n_slabs) indices,
 * one workgroup each, and top-k / top-p become the low edge of a bin of a
 * histogram of the weights (1024 bins uniform in -log w over [0, 40)), so the
 * kept set is the exact sampler's plus at most one bin (weights within a
 * factor e^(40/1024) = 1.04 below the exact threshold); min-p stays exact.
 * The draw is an exact function of (logits, seen, parameters, seed, n_slabs).
 * `work`: vpq_sample_hist_workspace_bytes(n_slabs) bytes of device scratch
 * (slab maxima, per-slab histograms, their sum, the threshold, per-slab
 * picks), 4-byte aligned; nothing in it needs to be cleared.
 * Requires 1 <= V <= 2^24, rep != 0, 1 <= n_slabs <= 1024, ceil(V / n_slabs) <= 65535
 * (the per-slab fixed-point masses); other requirements as above. */
size_t vpq_sample_hist_workspace_bytes(int n_slabs);
int vpq_sample_hist_bf16(vpq_stream_t stream, const uint16_t* logits, int32_t* out_id, int V, float temp,
                         float top_p, uint32_t seed, uint16_t* ws, float rep_penalty, float presence_penalty,
                         int top_k, float min_p, uint8_t* seen, int n_slabs, void* work, size_t work_bytes);

/* ---- measurement aid (no counterpart in the reference's kernels; the
 * reference times command buffers with Fence::gpu_times(),
 * apple-silicon/metal-compute/command-stream.h:119-126) -----------------------
 * vpq_profile_enable(n > 0): from now on each kernel the library launches is
 * bracketed by its own pair of HIP events (hipExtLaunchKernel start/stop), up to
 * n launches; n <= 0 switches it off.  vpq_profile_read() waits for the recorded
 * launches, writes each kernel's duration in milliseconds, in launch order, to
 * kernel_ms[0..capacity) and returns how many launches were recorded (or a
 * negative status), then starts over.  Not for use under graph capture.  The
 * recording state is shared and unsynchronised: while it is on, only one thread
 * may call into the library. */
int vpq_profile_enable(int max_launches);
int vpq_profile_read(float* kernel_ms, int capacity);
/* The yardsticks a benchmark times beside the product's kernels, in the same run and the same way: a kernel that
 * does nothing (launch + completion), and a kernel that only reads the first `bytes` (>= 16, a multiple of 16 is
 * read) of `src` with 16-byte loads, eight in flight per thread, all requested before the first is used.  `sink`
 * (4 bytes of device memory) is never written. */
int vpq_profile_empty_kernel(vpq_stream_t stream, void* sink);
int vpq_profile_read_kernel(vpq_stream_t stream, const void* src, size_t bytes, void* sink);

/* Output byte sizes of the packer (generative-models/quantize/affine-quantizer.h:37-40). */
size_t vpq_weight_bytes(int N, int K);
size_t vpq_scale_bytes(int N, int K);

#ifdef __cplusplus
}
#endif
#endif /* VPQ_H */

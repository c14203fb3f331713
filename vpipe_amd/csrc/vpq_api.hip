// The C ABI (include/vpq.h): argument validation, device check and kernel
// selection.  Nothing here allocates device memory or synchronises.
#include "../../include/vpq.h"

#include <hip/hip_runtime.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "vpq_internal.h"

namespace vpq {
ProfileState& profile_state()
{
  static ProfileState ps;
  return ps;
}
}  // namespace vpq

namespace {

struct DeviceState {
  std::atomic<int> status{1};  // 1 = not initialised, 0 = ok, <0 = vpq_status
  int cu_count = 0;
};

DeviceState g_dev;
std::mutex g_init_mutex;
thread_local char g_last_error[256] = "";

int device_error(hipError_t e)
{
  const char* s = hipGetErrorString(e);
  strncpy(g_last_error, s ? s : "unknown HIP error", sizeof(g_last_error) - 1);
  g_last_error[sizeof(g_last_error) - 1] = '\0';
  return VPQ_ERR_DEVICE;
}

int ensure_init()
{
  int st = g_dev.status.load(std::memory_order_acquire);
  if (st <= 0) { return st; }
  std::lock_guard<std::mutex> lock(g_init_mutex);
  st = g_dev.status.load(std::memory_order_acquire);
  if (st <= 0) { return st; }
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { return device_error(e); }
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) { return device_error(e); }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    strncpy(g_last_error, "device is not gfx950", sizeof(g_last_error) - 1);
    g_dev.status.store(VPQ_ERR_UNSUPPORTED, std::memory_order_release);
    return VPQ_ERR_UNSUPPORTED;
  }
  g_dev.cu_count = prop.multiProcessorCount;
  g_dev.status.store(VPQ_OK, std::memory_order_release);
  return VPQ_OK;
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

inline int finish(hipError_t e) { return e == hipSuccess ? VPQ_OK : device_error(e); }

int check_pack(const uint32_t* w, const uint16_t* scales, const uint16_t* biases, int K, int N)
{
  if (w == nullptr || scales == nullptr || biases == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (K <= 0 || N <= 0 || (K % 64) != 0) { return VPQ_ERR_BAD_SHAPE; }
  // Rows of codes are K/2 bytes, a multiple of 32: 16-byte alignment of the base
  // makes every 128-bit load of the kernels aligned.  Scales/biases are read
  // with 2-byte loads by the general kernels; the vector paths need 16.
  if (!aligned(w, 16) || !aligned(scales, 2) || !aligned(biases, 2)) { return VPQ_ERR_MISALIGNED; }
  return VPQ_OK;
}

// Rows from which the size-based entrance takes the dequant-once route when the workspace holds the
// expanded weight: the expansion costs ~20 us per 28 MB pack, the dense GEMM then runs ~1.1x faster than the
// fused kernel where the tiles are many (measured at M = 16320: 1.3 against 1.2 PFLOP/s; at M = 2048 the two
// are even on 4096->12288 and the fused kernel is ahead on the N = 4096 shapes).
constexpr int kDenseRouteMinRows = 8192;

int qmv_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
               const uint16_t* biases, const uint16_t* x, void* y, bool y_f32, int K, int N, int M,
               const uint16_t* residual, void* ws, size_t ws_bytes, int variant, int gate_act = 0)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 16) { return VPQ_ERR_BAD_SHAPE; }
  const bool gelu_mul = gate_act == vpq::kStoreGeluMul;       // `residual` is the multiplier [N]; bf16 store only
  if (gate_act != 0 && gate_act != VPQ_GATE_SWIGLU && gate_act != VPQ_GATE_GEGLU && !gelu_mul) { return VPQ_ERR_BAD_SHAPE; }
  if (gelu_mul && (residual == nullptr || y_f32 || variant != VPQ_QMV_AUTO)) { return residual == nullptr ? VPQ_ERR_NULL_POINTER : VPQ_ERR_BAD_SHAPE; }
  if (gate_act != 0 && !gelu_mul && ((N & 1) != 0 || residual != nullptr || variant == VPQ_QMV_STREAM)) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, y_f32 ? 4 : 2)) { return VPQ_ERR_MISALIGNED; }
  if (residual != nullptr && !aligned(residual, 2)) { return VPQ_ERR_MISALIGNED; }
  if (variant < VPQ_QMV_AUTO || variant > VPQ_QMV_RING_SPLITK || variant == 3) { return VPQ_ERR_BAD_SHAPE; }   // (3 is unassigned)
  st = ensure_init();
  if (st != VPQ_OK) { return st; }

  vpq::QmvArgs a;
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = y; a.residual = residual;
  a.K = K; a.N = N; a.M = M; a.y_f32 = y_f32; a.ws = ws; a.ws_bytes = ws_bytes;
  a.cu_count = g_dev.cu_count;
  a.gate_act = gate_act;
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);

  const bool mfma_ok = vpq::qmv_mfma_supports(K, N, M) && aligned(scales, 16) && aligned(biases, 16);
  const bool flow_ok = vpq::qmv_flow_supports(K, N, M) && aligned(scales, 16) && aligned(biases, 16);
  if (gelu_mul) {        // the two kernels that have this store: the streaming one and the general one
    return finish(flow_ok ? vpq::launch_qmv_flow(hs, a) : vpq::launch_qmv_simple(hs, a));
  }
  if (variant == VPQ_QMV_SIMPLE) { return finish(vpq::launch_qmv_simple(hs, a)); }
  if (variant == VPQ_QMV_FLOW) {
    if (!flow_ok) { return VPQ_ERR_BAD_SHAPE; }
    return finish(vpq::launch_qmv_flow(hs, a));
  }
  if (variant == VPQ_QMV_ROWS) {
    if (!vpq::qmv_rows_supports(K, N, M) || (gate_act != 0 && (N & 1) != 0)) { return VPQ_ERR_BAD_SHAPE; }
    return finish(vpq::launch_qmv_rows(hs, a, 0));
  }
  if (variant == VPQ_QMV_RING) {
    if (!mfma_ok || !vpq::qmv_ring_supports(K, N, M)) { return VPQ_ERR_BAD_SHAPE; }
    return finish(vpq::launch_qmv_ring(hs, a, 0, 1));
  }
  if (variant == VPQ_QMV_RING_SPLITK) {
    if (!mfma_ok || !vpq::qmv_ring_supports(K, N, M) || K < 1024) { return VPQ_ERR_BAD_SHAPE; }
    if (ws == nullptr || !aligned(ws, 16)) { return ws == nullptr ? VPQ_ERR_WORKSPACE : VPQ_ERR_MISALIGNED; }
    const int parts = K / 512 < 4 ? K / 512 : 4;
    if (ws_bytes < vpq::qmv_ring_workspace_bytes(K, N, M)) { return VPQ_ERR_WORKSPACE; }
    return finish(vpq::launch_qmv_ring(hs, a, 0, parts));
  }
  if (variant == VPQ_QMV_STREAM) {
    // handled below, after the shape check of the streaming kernel
  } else if (variant == VPQ_QMV_MFMA) {
    if (!mfma_ok) { return VPQ_ERR_BAD_SHAPE; }
    return finish(vpq::launch_qmv_mfma(hs, a));
  }
  const bool stream_ok = mfma_ok && gate_act == 0 && vpq::qmv_stream_supports(K, N, M);
  if (variant == VPQ_QMV_STREAM) {
    if (!stream_ok) { return VPQ_ERR_BAD_SHAPE; }
    return finish(vpq::launch_qmv_stream(hs, a));
  }
  // One row of x: the streaming kernel that requests the whole pack up front (measured, HBM-cold: 4096->12288
  // 6.8 us against 9.0 for the tile kernel, 4096->2x12288 11.5 against 15.6, the 5120->151936 lm_head 75.6 against
  // 79.7 for the persistent kernel below).
  if (flow_ok) { return finish(vpq::launch_qmv_flow(hs, a)); }
  // Two to four rows over an lm_head-sized pack: persistent workgroups that walk a tile's whole K.
  const double pack_bytes = (double)N * (double)K * 9.0 / 16.0;
  if (stream_ok && pack_bytes >= 150e6) { return finish(vpq::launch_qmv_stream(hs, a)); }
  // Several rows of x: the ring kernel keeps a slice of x in registers for all the tiles of a
  // workgroup (one workgroup per CU; it chooses its tiles per workgroup so that the launch runs in
  // few, full generations of workgroups), so x is re-read from L2 once per slice and workgroup instead
  // of once per item (measured at 16 rows: 117 vs 284 us at 5120->151936, 17.6 vs 39.9 us at
  // 5120->17408; at 4 rows 8.8 vs 12.0 us at 4096->12288; at 2 rows 15.1 vs 17.1 us at 5120->17408,
  // 16.0 vs 17.5 at 17408->5120).
  // (with a workspace the ring kernel splits K across workgroups where its cost model says that pays: many rows
  // over a deep K and a narrow N)
  if (mfma_ok && vpq::qmv_ring_supports(K, N, M) && M >= 2) {
    if (a.ws != nullptr && !aligned(a.ws, 16)) { a.ws = nullptr; a.ws_bytes = 0; }
    return finish(vpq::launch_qmv_ring(hs, a, 0, 0));
  }
  if (mfma_ok) { return finish(vpq::launch_qmv_mfma(hs, a)); }
  // K not a multiple of 512, or scales / biases off 16-byte alignment: the row-streaming kernel
  // for up to two rows of x, the general one above.
  if (vpq::qmv_rows_supports(K, N, M)) { return finish(vpq::launch_qmv_rows(hs, a, 0)); }
  return finish(vpq::launch_qmv_simple(hs, a));
}

}  // namespace

extern "C" {

int vpq_version(void) { return 100; }

const char* vpq_status_string(int status)
{
  switch (status) {
    case VPQ_OK: return "ok";
    case VPQ_ERR_NULL_POINTER: return "a required buffer is NULL";
    case VPQ_ERR_BAD_SHAPE: return "shape outside the supported domain";
    case VPQ_ERR_MISALIGNED: return "pointer not aligned as required";
    case VPQ_ERR_WORKSPACE: return "workspace missing or too small";
    case VPQ_ERR_DEVICE: return "HIP runtime error";
    case VPQ_ERR_UNSUPPORTED: return "device is not gfx950";
    default: return "unknown status";
  }
}

const char* vpq_last_device_error(void) { return g_last_error; }

int vpq_init(void)
{
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  // Also resolves the static scratch of vpq_argmax_bf16_static for the current device, so that the entry point
  // itself has no first-call work left.  Best effort: a failure here concerns that one entry point only, which
  // tries again on its first call and reports it there.
  float* unused = nullptr;
  (void)vpq::argmax_static_scratch(&unused);
  return VPQ_OK;
}

int vpq_device_cu_count(void) { return g_dev.status.load() == VPQ_OK ? g_dev.cu_count : 0; }

int vpq_dequant_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, uint16_t* w_deq, int K, int N)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (w_deq == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (!aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_dequant(reinterpret_cast<hipStream_t>(stream), w, scales, biases, w_deq, K, N));
}

int vpq_dequant_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, uint16_t* w_deq, int K, int N)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (w_deq == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (!aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_dequant8(reinterpret_cast<hipStream_t>(stream), w, scales, biases, w_deq, K, N));
}

static int qmv8_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       const uint16_t* x, void* y, bool y_f32, int K, int N, int M, const uint16_t* residual,
                       int store = 0)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr || (store == vpq::kStoreGeluMul && residual == nullptr)) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 16) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, y_f32 ? 4 : 2) || (residual != nullptr && !aligned(residual, 2))) {
    return VPQ_ERR_MISALIGNED;
  }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = y; a.residual = residual;
  a.K = K; a.N = N; a.M = M; a.y_f32 = y_f32; a.cu_count = g_dev.cu_count;
  a.gate_act = store;
  return finish(vpq::launch_qmv_simple8(reinterpret_cast<hipStream_t>(stream), a));
}

int vpq_qmv_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       const uint16_t* x, uint16_t* y, int K, int N, int M, const uint16_t* residual)
{
  return qmv8_common(stream, w, scales, biases, x, y, false, K, N, M, residual);
}

int vpq_qmv_w8g64_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                         const uint16_t* x, float* y, int K, int N, int M)
{
  return qmv8_common(stream, w, scales, biases, x, y, true, K, N, M, nullptr);
}

int vpq_qmv_gelu_mul_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                                const uint16_t* x, uint16_t* y, int K, int N, const uint16_t* mul)
{
  return qmv8_common(stream, w, scales, biases, x, y, false, K, N, 1, mul, vpq::kStoreGeluMul);
}

int vpq_moe_gate_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            const uint16_t* x, uint16_t* gate, int K, int M)
{
  int st = check_pack(w, scales, biases, K, 1);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || gate == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 65535) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(gate, 2)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = gate;
  a.K = K; a.N = 1; a.M = 1; a.y_f32 = false; a.cu_count = g_dev.cu_count;
  a.gate_act = vpq::kStoreSigmoid;
  return finish(vpq::launch_qmv_rows8(reinterpret_cast<hipStream_t>(stream), a, M, nullptr, 1, 1));
}

static int rows8_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                        const uint16_t* x, uint16_t* y, int K, int N, int rows, int gate_act, const int32_t* pair_eid,
                        bool gathered, int x_div, int n_experts)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr || (gathered && pair_eid == nullptr)) { return VPQ_ERR_NULL_POINTER; }
  if (gate_act != 0 && gate_act != VPQ_GATE_SWIGLU && gate_act != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (rows < 1 || rows > 65535 || (gate_act != 0 && (N & 1) != 0)) { return VPQ_ERR_BAD_SHAPE; }
  if (gathered ? (x_div < 1 || n_experts < 1) : rows > 16) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 2) || (gathered && !aligned(pair_eid, 4))) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = y;
  a.K = K; a.N = N; a.M = 1; a.y_f32 = false; a.cu_count = g_dev.cu_count;
  a.gate_act = gate_act;
  return finish(vpq::launch_qmv_rows8(reinterpret_cast<hipStream_t>(stream), a, rows, gathered ? pair_eid : nullptr, x_div,
                                      n_experts));
}

int vpq_gather_qmv_gated_split_bf16(vpq_stream_t stream, const uint32_t* wg, const uint16_t* sg, const uint16_t* bg,
                                    int gate_bits, const uint32_t* wu, const uint16_t* su, const uint16_t* bu, int up_bits,
                                    const uint16_t* x, uint16_t* y, int K, int ffn, const int32_t* pair_eid, int npair,
                                    int top_k, int n_experts, int activation)
{
  if (wg == nullptr || sg == nullptr || bg == nullptr || wu == nullptr || su == nullptr || bu == nullptr || x == nullptr ||
      y == nullptr) {
    return VPQ_ERR_NULL_POINTER;
  }
  if ((gate_bits != 4 && gate_bits != 8) || (up_bits != 4 && up_bits != 8)) { return VPQ_ERR_BAD_SHAPE; }
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (K <= 0 || (K % 64) != 0 || ffn < 1 || npair < 1 || npair > 65535) { return VPQ_ERR_BAD_SHAPE; }
  if (pair_eid != nullptr ? (top_k < 1 || n_experts < 1) : npair > 16) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(wg, 16) || !aligned(wu, 16) || !aligned(x, 16) || !aligned(sg, 2) || !aligned(bg, 2) || !aligned(su, 2) ||
      !aligned(bu, 2) || !aligned(y, 2) || (pair_eid != nullptr && !aligned(pair_eid, 4))) {
    return VPQ_ERR_MISALIGNED;
  }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::SplitGateUp a{};
  a.wg = wg; a.sg = sg; a.bg = bg; a.gate_bits = gate_bits;
  a.wu = wu; a.su = su; a.bu = bu; a.up_bits = up_bits;
  a.x = x; a.y = y; a.K = K; a.F = ffn; a.rows = npair; a.gate_act = activation;
  a.pair_eid = pair_eid; a.x_div = pair_eid != nullptr ? top_k : 1; a.n_experts = n_experts;
  return finish(vpq::launch_qmv_split_gate_up(reinterpret_cast<hipStream_t>(stream), a));
}

int vpq_qmv_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, uint16_t* y, int K, int N, int M, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return rows8_common(stream, w, scales, biases, x, y, K, N, M, activation, nullptr, false, 1, 1);
}

int vpq_gather_qmv_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                    const int32_t* pair_eid, int npair, int top_k, int n_experts, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return rows8_common(stream, w, scales, biases, x, y, K, N, npair, activation, pair_eid, true, top_k, n_experts);
}

int vpq_gather_down_qmv_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                   const int32_t* pair_eid, int npair, int n_experts)
{
  return rows8_common(stream, w, scales, biases, x, y, K, N, npair, 0, pair_eid, true, 1, n_experts);
}

int vpq_qmm_dense_route_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                   uint16_t* w_deq, int expand)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (w_deq == nullptr) { return VPQ_ERR_WORKSPACE; }
  if (M <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16) || !aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (expand != 0) {
    st = finish(vpq::launch_dequant8(hs, w, scales, biases, w_deq, K, N));
    if (st != VPQ_OK) { return st; }
  }
  std::string why;
  const int rc = vpq::dense_gemm_bf16(hs, x, w_deq, y, M, N, K, g_dev.cu_count, &why);
  if (rc != 0) {
    strncpy(g_last_error, why.c_str(), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return VPQ_ERR_DEVICE;
  }
  return VPQ_OK;
}

// ---- 8-bit codes in groups of 32 (GGUF q8 repacked; the codec's int8 path): `affine_dequant_w8g32`
// (affine_dequant.metal:99-131), `affine_qmv_w8g32` (affine_qmv.metal:3053-3069), `affine_qmm_steel_w8g32`
// (affine_qmm_steel.metal:1674-1698) by the dequant-once route, which is how the reference's codec runs it.
namespace {

int check_pack_w8g32(const uint32_t* w, const uint16_t* scales, const uint16_t* biases, int K, int N)
{
  if (w == nullptr || scales == nullptr || biases == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (K <= 0 || N <= 0 || (K % 32) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(w, 16) || !aligned(scales, 2) || !aligned(biases, 2)) { return VPQ_ERR_MISALIGNED; }
  return VPQ_OK;
}

}  // namespace

int vpq_dequant_w8g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           uint16_t* w_deq, int K, int N)
{
  int st = check_pack_w8g32(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (w_deq == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (!aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_dequant8(reinterpret_cast<hipStream_t>(stream), w, scales, biases, w_deq, K, N, 32));
}

int vpq_requant_w8_to_w4_g64_bf16(vpq_stream_t stream, const uint32_t* w8, const uint16_t* s8, const uint16_t* b8,
                                  uint32_t* w4, uint16_t* s4, uint16_t* b4, int K, int N)
{
  int st = check_pack(w8, s8, b8, K, N);
  if (st != VPQ_OK) { return st; }
  if (w4 == nullptr || s4 == nullptr || b4 == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (!aligned(w4, 16) || !aligned(s4, 2) || !aligned(b4, 2)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_requant_w8_to_w4(reinterpret_cast<hipStream_t>(stream), w8, s8, b8, w4, s4, b4, K, N));
}

int vpq_qmv_w8g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       const uint16_t* x, uint16_t* y, int K, int N, int M, const uint16_t* residual)
{
  int st = check_pack_w8g32(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 16 || (K % 16) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 2) || (residual != nullptr && !aligned(residual, 2))) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = y; a.residual = residual;
  a.K = K; a.N = N; a.M = M; a.y_f32 = false; a.cu_count = g_dev.cu_count;
  return finish(vpq::launch_qmv_simple8(reinterpret_cast<hipStream_t>(stream), a, 32));
}

int vpq_qmm_dense_route_w8g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                   uint16_t* w_deq, int expand)
{
  int st = check_pack_w8g32(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (w_deq == nullptr) { return VPQ_ERR_WORKSPACE; }
  if (M <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16) || !aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (expand != 0) {
    st = finish(vpq::launch_dequant8(hs, w, scales, biases, w_deq, K, N, 32));
    if (st != VPQ_OK) { return st; }
  }
  std::string why;
  const int rc = vpq::dense_gemm_bf16(hs, x, w_deq, y, M, N, K, g_dev.cu_count, &why);
  if (rc != 0) {
    strncpy(g_last_error, why.c_str(), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return VPQ_ERR_DEVICE;
  }
  return VPQ_OK;
}

int vpq_embed_gather_w4g64_bf16(vpq_stream_t stream, const int32_t* ids, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, uint16_t* out, int H, int T, int vocab)
{
  int st = check_pack(w, scales, biases, H, vocab);
  if (st != VPQ_OK) { return st; }
  if (ids == nullptr || out == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (T <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(ids, 4) || !aligned(out, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_embed_gather(reinterpret_cast<hipStream_t>(stream), ids, w, scales, biases, out, H, T, vocab));
}

int vpq_qmv_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                       const uint16_t* residual, void* ws, size_t ws_bytes, int variant)
{
  return qmv_common(stream, w, scales, biases, x, y, false, K, N, M, residual, ws, ws_bytes, variant);
}

int vpq_qmv_w4g64_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                         const uint16_t* biases, const uint16_t* x, float* y, int K, int N, int M,
                         void* ws, size_t ws_bytes, int variant)
{
  return qmv_common(stream, w, scales, biases, x, y, true, K, N, M, nullptr, ws, ws_bytes, variant);
}

size_t vpq_qmv_workspace_bytes(int K, int N, int M)
{
  if (K <= 0 || N <= 0 || M < 1 || M > 16) { return 0; }
  return (vpq::qmv_ring_workspace_bytes(K, N, M) + 255) / 256 * 256;
}

int vpq_lora_a_bf16(vpq_stream_t stream, const uint16_t* x, const uint16_t* lora_a, uint16_t* t,
                    int M, int K, int r, float alpha)
{
  if (x == nullptr || lora_a == nullptr || t == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M <= 0 || K <= 0 || (K % 64) != 0 || r < 8 || r > vpq::kLoraMaxRank || (r % 8) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(lora_a, 16) || !aligned(t, 16)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_lora_a(reinterpret_cast<hipStream_t>(stream), x, lora_a, t, M, K, r, alpha));
}

namespace {

// tile: 0 = by size, 128 = the 256 x 128 tile kernel, 192 / 256 = the large-tile kernel at that width,
// -128 = the large-tile kernel at width 128
int qmm_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
               const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
               const uint16_t* lora_a, const uint16_t* lora_b, int r, float alpha,
               uint16_t* lora_t_ws, int tile)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16)) { return VPQ_ERR_MISALIGNED; }
  const bool lora = lora_a != nullptr && alpha != 0.0f;
  if (lora) {
    if (lora_b == nullptr) { return VPQ_ERR_NULL_POINTER; }
    if (lora_t_ws == nullptr) { return VPQ_ERR_WORKSPACE; }
    if (r < 8 || r > vpq::kLoraMaxRank || (r % 8) != 0) { return VPQ_ERR_BAD_SHAPE; }
    if (!aligned(lora_a, 16) || !aligned(lora_b, 16) || !aligned(lora_t_ws, 16)) { return VPQ_ERR_MISALIGNED; }
  }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (lora) {
    st = vpq_lora_a_bf16(stream, x, lora_a, lora_t_ws, M, K, r, alpha);
    if (st != VPQ_OK) { return st; }
  }
  vpq::GemmArgs g{};
  g.w = w; g.scales = scales; g.biases = biases; g.x = x; g.y = y;
  g.K = K; g.N = N; g.M = M;
  g.lora_t = lora ? lora_t_ws : nullptr;
  g.lora_b = lora ? lora_b : nullptr;
  g.r = lora ? r : 0;
  g.cu_count = g_dev.cu_count;
  if (tile == 192 || tile == 256 || tile == -128) {
    if (!vpq::qmm_big_supports(g)) { return VPQ_ERR_BAD_SHAPE; }
    return finish(vpq::launch_qmm_big(hs, g, tile < 0 ? -tile : tile));
  }
  // The large-tile kernel once its tiles fill the CUs at least once (measured: 1.02-1.16 against
  // 0.83-0.91 PFLOP/s at M = 16320, 0.98 against 0.78 at 4096 -> 12288 and 0.94 against 0.91 at
  // 12288 -> 4096 with M = 2048); with fewer tiles the two are equal and the tile kernel has the
  // split-K form beside it.
  if (tile == 0 && vpq::qmm_big_supports(g)) {
    const int bn = vpq::qmm_big_tile_n(N, M, g_dev.cu_count);
    const long tiles = (long)((M + 255) / 256) * (long)((N + bn - 1) / bn);
    if (tiles >= (long)(g_dev.cu_count > 0 ? g_dev.cu_count : 256)) { return finish(vpq::launch_qmm_big(hs, g, bn)); }
  }
  return finish(vpq::launch_qmm_tile(hs, g));
}

}  // namespace

int vpq_qmm_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                       const uint16_t* lora_a, const uint16_t* lora_b, int r, float alpha,
                       uint16_t* lora_t_ws)
{
  return qmm_common(stream, w, scales, biases, x, y, K, N, M, lora_a, lora_b, r, alpha, lora_t_ws, 0);
}

int vpq_qmm_tiled_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                             const uint16_t* lora_a, const uint16_t* lora_b, int r, float alpha,
                             uint16_t* lora_t_ws, int tile_n)
{
  if (tile_n != 128 && tile_n != -128 && tile_n != 192 && tile_n != 256) { return VPQ_ERR_BAD_SHAPE; }
  return qmm_common(stream, w, scales, biases, x, y, K, N, M, lora_a, lora_b, r, alpha, lora_t_ws, tile_n);
}

size_t vpq_linear_workspace_bytes(int K, int N, int M)
{
  if (K <= 0 || N <= 0 || M <= 0 || (K % 64) != 0) { return 0; }
  if (M >= kDenseRouteMinRows) { return ((size_t)N * (size_t)K * 2 + 255) / 256 * 256; }
  return vpq_qmm_workspace_bytes(K, N, M);
}

size_t vpq_qmm_workspace_bytes(int K, int N, int M)
{
  if (K <= 0 || N <= 0 || M <= 0 || (K % 64) != 0) { return 0; }
  if (ensure_init() != VPQ_OK) { return 0; }
  return (vpq::qmm_splitk_workspace_bytes(K, N, M, g_dev.cu_count) + 255) / 256 * 256;
}

int vpq_qmm_splitk_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                              int splits, void* ws, size_t ws_bytes)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M <= 0 || splits < 0 || splits > 16) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16) || (ws != nullptr && !aligned(ws, 256))) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  if (splits == 0) { splits = vpq::qmm_choose_splits(K, N, M, g_dev.cu_count); }
  if (splits > K / 64) { splits = K / 64; }
  vpq::GemmArgs g{};
  g.w = w; g.scales = scales; g.biases = biases; g.x = x; g.y = y;
  g.K = K; g.N = N; g.M = M;
  g.cu_count = g_dev.cu_count;
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (splits <= 1) { return finish(vpq::launch_qmm_tile(hs, g)); }
  if (ws == nullptr || ws_bytes < (size_t)splits * (size_t)M * (size_t)N * sizeof(float)) { return VPQ_ERR_WORKSPACE; }
  return finish(vpq::launch_qmm_tile_splitk(hs, g, splits, static_cast<float*>(ws)));
}

int vpq_qmm_dense_route_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                   uint16_t* w_deq, int expand)
{
  return vpq_qmm_dense_route_lora_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, w_deq, expand, nullptr, nullptr, 0,
                                             0.0f, nullptr);
}

// The dequant-once route with the runtime adapter: the pre-pass t = bf16(alpha * bf16(x . A^T)), the expansion (or the
// kept one), then the dense GEMM with t . B^T in the same accumulators -- the bits of vpq_qmm_w4g64_bf16 with the
// same adapter.
int vpq_qmm_dense_route_lora_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                        const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                        uint16_t* w_deq, int expand, const uint16_t* lora_a, const uint16_t* lora_b,
                                        int r, float alpha, uint16_t* lora_t_ws)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (w_deq == nullptr) { return VPQ_ERR_WORKSPACE; }
  if (M <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16) || !aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  const bool lora = lora_a != nullptr && alpha != 0.0f;
  if (lora) {
    if (lora_b == nullptr) { return VPQ_ERR_NULL_POINTER; }
    if (lora_t_ws == nullptr) { return VPQ_ERR_WORKSPACE; }
    if (r < 8 || r > vpq::kLoraMaxRank || (r % 8) != 0) { return VPQ_ERR_BAD_SHAPE; }
    if (!aligned(lora_a, 16) || !aligned(lora_b, 16) || !aligned(lora_t_ws, 16)) { return VPQ_ERR_MISALIGNED; }
  }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (lora) {
    st = finish(vpq::launch_lora_a(hs, x, lora_a, lora_t_ws, M, K, r, alpha));
    if (st != VPQ_OK) { return st; }
  }
  if (expand != 0) {
    st = finish(vpq::launch_dequant(hs, w, scales, biases, w_deq, K, N));
    if (st != VPQ_OK) { return st; }
  }
  std::string why;
  const int rc = vpq::dense_gemm_elt(hs, x, w_deq, y, M, N, K, false, g_dev.cu_count, &why, lora ? lora_t_ws : nullptr,
                                     lora ? lora_b : nullptr, lora ? r : 0);
  if (rc != 0) {
    strncpy(g_last_error, why.c_str(), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return VPQ_ERR_DEVICE;
  }
  return VPQ_OK;
}

// ---- IEEE binary16 element type (VPIPE_ELT = half) ----

int vpq_dequant_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                          uint16_t* w_deq, int K, int N)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (w_deq == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (!aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_dequant_f16(reinterpret_cast<hipStream_t>(stream), w, scales, biases, w_deq, K, N));
}

static int qmv_f16_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                          const uint16_t* x, void* y, bool y_f32, int K, int N, int M, const uint16_t* residual,
                          int gate_act)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 16) { return VPQ_ERR_BAD_SHAPE; }
  if (gate_act != 0 && ((N & 1) != 0 || residual != nullptr)) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, y_f32 ? 4 : 2) || (residual != nullptr && !aligned(residual, 2))) {
    return VPQ_ERR_MISALIGNED;
  }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = y; a.residual = residual;
  a.K = K; a.N = N; a.M = M; a.y_f32 = y_f32; a.cu_count = g_dev.cu_count;
  a.gate_act = gate_act;
  // one row of x on a K the streaming kernel takes: the same kernel as for bf16, on binary16 arithmetic
  if (vpq::qmv_flow_supports(K, N, M) && aligned(scales, 16) && aligned(biases, 16)) {
    return finish(vpq::launch_qmv_flow_f16(reinterpret_cast<hipStream_t>(stream), a));
  }
  // several rows (K % 512 == 0): the kernels of the bf16 entry on binary16 arithmetic -- two to four rows over an
  // lm_head-sized pack the streaming kernel, otherwise the ring kernel
  const bool tuned = M >= 2 && vpq::qmv_mfma_supports(K, N, M) && aligned(scales, 16) && aligned(biases, 16);
  if (tuned && gate_act == 0 && vpq::qmv_stream_supports(K, N, M) && (double)N * (double)K * 9.0 / 16.0 >= 150e6) {
    return finish(vpq::launch_qmv_stream(reinterpret_cast<hipStream_t>(stream), a, true));
  }
  if (tuned && vpq::qmv_ring_supports(K, N, M)) {
    return finish(vpq::launch_qmv_ring(reinterpret_cast<hipStream_t>(stream), a, 0, 0, true));
  }
  return finish(vpq::launch_qmv_simple_f16(reinterpret_cast<hipStream_t>(stream), a));
}

int vpq_qmv_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                      const uint16_t* x, uint16_t* y, int K, int N, int M, const uint16_t* residual)
{
  return qmv_f16_common(stream, w, scales, biases, x, y, false, K, N, M, residual, 0);
}

int vpq_qmv_w4g64_f16_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, float* y, int K, int N, int M)
{
  return qmv_f16_common(stream, w, scales, biases, x, y, true, K, N, M, nullptr, 0);
}

int vpq_qmv_gated_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                            const uint16_t* x, uint16_t* y, int K, int N, int M, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return qmv_f16_common(stream, w, scales, biases, x, y, false, K, N, M, nullptr, activation);
}

namespace {

// The fused GEMM on binary16 elements: the large-tile kernel once its tiles fill the CUs (K % 512 == 0, 16-byte
// aligned scales and biases), the 256 x 128 tile kernel otherwise -- same MFMA, same K order, same bits.
// activation 0 = plain y [M,N], else the gated store of an interleaved gate|up pack, y [M,N/2] (no adapter then).
int qmm_f16_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, uint16_t* y, int K, int N, int M, int activation, const uint16_t* lora_a,
                   const uint16_t* lora_b, int r, float alpha, uint16_t* lora_t_ws)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (activation != 0 && activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (M <= 0 || (activation != 0 && (N & 1) != 0)) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16)) { return VPQ_ERR_MISALIGNED; }
  const bool lora = lora_a != nullptr && alpha != 0.0f;
  if (lora) {
    if (activation != 0) { return VPQ_ERR_BAD_SHAPE; }
    if (lora_b == nullptr) { return VPQ_ERR_NULL_POINTER; }
    if (lora_t_ws == nullptr) { return VPQ_ERR_WORKSPACE; }
    if (r < 8 || r > vpq::kLoraMaxRank || (r % 8) != 0) { return VPQ_ERR_BAD_SHAPE; }
    if (!aligned(lora_a, 16) || !aligned(lora_b, 16) || !aligned(lora_t_ws, 16)) { return VPQ_ERR_MISALIGNED; }
  }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (lora) {
    st = finish(vpq::launch_lora_a(hs, x, lora_a, lora_t_ws, M, K, r, alpha, true));
    if (st != VPQ_OK) { return st; }
  }
  vpq::GemmArgs g{};
  g.w = w; g.scales = scales; g.biases = biases; g.x = x; g.y = y;
  g.K = K; g.N = N; g.M = M;
  g.lora_t = lora ? lora_t_ws : nullptr;
  g.lora_b = lora ? lora_b : nullptr;
  g.r = lora ? r : 0;
  g.cu_count = g_dev.cu_count;
  g.gate_act = activation;
  g.f16 = true;
  if (vpq::qmm_big_supports(g)) {
    const int bn = vpq::qmm_big_tile_n(N, M, g_dev.cu_count);
    const long tiles = (long)((M + 255) / 256) * (long)((N + bn - 1) / bn);
    if (tiles >= (long)(g_dev.cu_count > 0 ? g_dev.cu_count : 256)) { return finish(vpq::launch_qmm_big(hs, g, bn)); }
  }
  return finish(vpq::launch_qmm_tile(hs, g));
}

}  // namespace

int vpq_qmm_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                      const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M, int activation)
{
  return qmm_f16_common(stream, w, scales, biases, x, y, K, N, M, activation, nullptr, nullptr, 0, 0.0f, nullptr);
}

int vpq_lora_a_f16(vpq_stream_t stream, const uint16_t* x, const uint16_t* lora_a, uint16_t* t, int M, int K, int r,
                   float alpha)
{
  if (x == nullptr || lora_a == nullptr || t == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M <= 0 || K <= 0 || (K % 64) != 0 || r < 8 || r > vpq::kLoraMaxRank || (r % 8) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(lora_a, 16) || !aligned(t, 16)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_lora_a(reinterpret_cast<hipStream_t>(stream), x, lora_a, t, M, K, r, alpha, true));
}

// The same with a runtime adapter: the pre-pass t = f16(alpha * f16(x . A^T)), then r more values of K from t and B
// in the GEMM's accumulators.  alpha == 0 or lora_a == NULL: no adapter.
int vpq_qmm_lora_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           const uint16_t* x, uint16_t* y, int K, int N, int M, const uint16_t* lora_a,
                           const uint16_t* lora_b, int r, float alpha, uint16_t* lora_t_ws)
{
  return qmm_f16_common(stream, w, scales, biases, x, y, K, N, M, 0, lora_a, lora_b, r, alpha, lora_t_ws);
}

int vpq_qmm_dense_route_w4g64_f16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                  const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                  uint16_t* w_deq, int expand)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (w_deq == nullptr) { return VPQ_ERR_WORKSPACE; }
  if (M <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16) || !aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (expand != 0) {
    st = finish(vpq::launch_dequant_f16(hs, w, scales, biases, w_deq, K, N));
    if (st != VPQ_OK) { return st; }
  }
  std::string why;
  const int rc = vpq::dense_gemm_elt(hs, x, w_deq, y, M, N, K, true, g_dev.cu_count, &why);
  if (rc != 0) {
    strncpy(g_last_error, why.c_str(), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return VPQ_ERR_DEVICE;
  }
  return VPQ_OK;
}

// Rows up to which the size-based entrances run the GEMV arithmetic in slabs of 16 rows instead of
// the 256-row GEMM tile: below it the tile kernel has one row of tiles and N/128 workgroups, and
// its time is its K loop's latency (57 us at 4096->4096 for any M <= 256) against ~10 us per slab.
constexpr int kSlabPlanMaxRows = 64;
constexpr int kSlabPlanSplitRows = 32;   // above: the split-K GEMM instead, when the workspace has the room

int vpq_linear_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                          const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                          void* ws, size_t ws_bytes)
{
  if (M >= 1 && M <= kSlabPlanMaxRows && x != nullptr && y != nullptr && K > 0 && N > 0) {
    // Three or four slabs: the GEMM with K split over the workgroups is faster where the workspace lets it
    // split (measured at 64 rows: 40 / 34 / 21 us against 43 / 68 / 31 us for four slabs at
    // 4096->12288 / 12288->4096 / 4096->4096; two slabs, 23 / 35 / 16 us, stay ahead of it).
    bool split_gemm = false;
    if (M > kSlabPlanSplitRows && ws != nullptr && aligned(ws, 256) && (K % 64) == 0 && ensure_init() == VPQ_OK) {
      const int splits = vpq::qmm_choose_splits(K, N, M, g_dev.cu_count);
      split_gemm = splits > 1 && ws_bytes >= (size_t)splits * (size_t)M * (size_t)N * sizeof(float);
    }
    if (!split_gemm) {
      for (int m0 = 0; m0 < M; m0 += 16) {
        const int rows = M - m0 < 16 ? M - m0 : 16;
        const int st = vpq_qmv_w4g64_bf16(stream, w, scales, biases, x + (size_t)m0 * K, y + (size_t)m0 * N, K, N, rows,
                                          nullptr, ws, ws_bytes, VPQ_QMV_AUTO);
        if (st != VPQ_OK) { return st; }
      }
      return VPQ_OK;
    }
  }
  // Very many rows: expanding the pack once into the workspace and running the dense GEMM on it beats the
  // fused kernels, the reference's own route for large M
  // (generative-models/minimax-h3/metal-minimax-h3-transformer.cc:2020-2160).
  if (ws != nullptr && aligned(ws, 256) && M >= kDenseRouteMinRows && K > 0 && N > 0 && (K % 64) == 0 &&
      ws_bytes >= (size_t)N * (size_t)K * 2 && vpq::dense_gemm_supports(M, N, K)) {
    return vpq_qmm_dense_route_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, static_cast<uint16_t*>(ws), 1);
  }
  // Few tiles and a long K: split K over more workgroups when the caller's workspace has the room.
  if (ws != nullptr && aligned(ws, 256) && K > 0 && N > 0 && M > 0 && (K % 64) == 0 && ensure_init() == VPQ_OK) {
    const int splits = vpq::qmm_choose_splits(K, N, M, g_dev.cu_count);
    if (splits > 1 && ws_bytes >= (size_t)splits * (size_t)M * (size_t)N * sizeof(float)) {
      return vpq_qmm_splitk_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, splits, ws, ws_bytes);
    }
  }
  return vpq_qmm_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, nullptr, nullptr, 0, 0.0f, nullptr);
}

int vpq_interleave_rows(vpq_stream_t stream, const void* a, const void* b, void* out, size_t row_bytes, size_t rows)
{
  if (a == nullptr || b == nullptr || out == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (row_bytes == 0 || (row_bytes & 1) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(a, 2) || !aligned(b, 2) || !aligned(out, 2)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_interleave_rows(reinterpret_cast<hipStream_t>(stream), a, b, out, row_bytes, rows));
}

int vpq_qmv_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                             int variant, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return qmv_common(stream, w, scales, biases, x, y, false, K, N, M, nullptr, nullptr, 0, variant, activation);
}

int vpq_qmv_gelu_mul_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                const uint16_t* mul)
{
  return qmv_common(stream, w, scales, biases, x, y, false, K, N, 1, mul, nullptr, 0, VPQ_QMV_AUTO, vpq::kStoreGeluMul);
}

int vpq_qmv_gated_w4g64_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                               const uint16_t* biases, const uint16_t* x, float* y, int K, int N, int M,
                               int variant, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return qmv_common(stream, w, scales, biases, x, y, true, K, N, M, nullptr, nullptr, 0, variant, activation);
}

int vpq_qmm_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                             const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                             int out_stride, int out_off, int activation)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (M <= 0 || (N & 1) != 0 || out_off < 0) { return VPQ_ERR_BAD_SHAPE; }
  if (out_stride > 0 && out_off + N / 2 > out_stride) { return VPQ_ERR_BAD_SHAPE; }
  if (out_stride <= 0 && out_off != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::GemmArgs g{};
  g.w = w; g.scales = scales; g.biases = biases; g.x = x; g.y = y;
  g.K = K; g.N = N; g.M = M;
  g.cu_count = g_dev.cu_count;
  g.gate_act = activation;
  g.out_stride = out_stride;
  g.out_off = out_off;
  // as vpq_qmm_w4g64_bf16: the large-tile kernel once its tiles fill the CUs (bit-identical results)
  if (vpq::qmm_big_supports(g)) {
    const int bn = vpq::qmm_big_tile_n(N, M, g_dev.cu_count);
    const long tiles = (long)((M + 255) / 256) * (long)((N + bn - 1) / bn);
    if (tiles >= (long)(g_dev.cu_count > 0 ? g_dev.cu_count : 256)) {
      return finish(vpq::launch_qmm_big(reinterpret_cast<hipStream_t>(stream), g, bn));
    }
  }
  return finish(vpq::launch_qmm_tile(reinterpret_cast<hipStream_t>(stream), g));
}

int vpq_linear_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                int activation)
{
  if (M >= 1 && M <= kSlabPlanMaxRows && x != nullptr && y != nullptr && K > 0 && N > 0) {
    for (int m0 = 0; m0 < M; m0 += 16) {
      const int rows = M - m0 < 16 ? M - m0 : 16;
      const int st = vpq_qmv_gated_w4g64_bf16(stream, w, scales, biases, x + (size_t)m0 * K, y + (size_t)m0 * (N / 2), K, N,
                                              rows, VPQ_QMV_AUTO, activation);
      if (st != VPQ_OK) { return st; }
    }
    return VPQ_OK;
  }
  return vpq_qmm_gated_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, 0, 0, activation);
}

int vpq_qmv_swiglu_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                              int variant)
{
  return vpq_qmv_gated_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, variant, VPQ_GATE_SWIGLU);
}

int vpq_qmv_swiglu_w4g64_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                const uint16_t* biases, const uint16_t* x, float* y, int K, int N, int M,
                                int variant)
{
  return vpq_qmv_gated_w4g64_f32out(stream, w, scales, biases, x, y, K, N, M, variant, VPQ_GATE_SWIGLU);
}

int vpq_qmm_swiglu_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                              int out_stride, int out_off)
{
  return vpq_qmm_gated_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, out_stride, out_off, VPQ_GATE_SWIGLU);
}

int vpq_linear_swiglu_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                 const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M)
{
  return vpq_linear_gated_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, VPQ_GATE_SWIGLU);
}

namespace {

int gather_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                  const uint16_t* x, uint16_t* y, int K, int N, const int32_t* pair_eid, int npair, int x_div,
                  int n_experts, int gate_act)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr || pair_eid == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (npair < 1 || npair > 65535 || x_div < 1 || n_experts < 1) { return VPQ_ERR_BAD_SHAPE; }
  if (gate_act != 0 && (N & 1) != 0) { return VPQ_ERR_BAD_SHAPE; }
  // every slab and every row of x must keep the 16-byte alignment of the base
  if (!aligned(x, 16) || !aligned(y, 2) || !aligned(pair_eid, 4)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = y;
  a.K = K; a.N = N; a.M = 1; a.y_f32 = false; a.cu_count = g_dev.cu_count;
  a.gate_act = gate_act;
  return finish(vpq::launch_qmv_rows_gather(reinterpret_cast<hipStream_t>(stream), a, pair_eid, npair, x_div, n_experts));
}

}  // namespace

int vpq_gather_qmv_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                    const int32_t* pair_eid, int npair, int top_k, int n_experts, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return gather_common(stream, w, scales, biases, x, y, K, N, pair_eid, npair, top_k, n_experts, activation);
}

int vpq_gather_down_qmv_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                   const int32_t* pair_eid, int npair, int n_experts)
{
  return gather_common(stream, w, scales, biases, x, y, K, N, pair_eid, npair, 1, n_experts, 0);
}

namespace {

int sorted_qmv_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                      const uint16_t* x, uint16_t* y, int K, int N, int npad, const int32_t* tile2e, const int32_t* srow,
                      int n_experts, int gate_act, bool x_from_srow, int bits = 4)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr || tile2e == nullptr || srow == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (npad < VPQ_QMV_GROUPED_SLOTS || (npad % VPQ_QMV_GROUPED_SLOTS) != 0 || npad / VPQ_QMV_GROUPED_SLOTS > 65535 ||
      n_experts < 1) {
    return VPQ_ERR_BAD_SHAPE;
  }
  if (gate_act != 0 && gate_act != VPQ_GATE_SWIGLU && gate_act != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (gate_act != 0 && (N & 1) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 2) || !aligned(tile2e, 4) || !aligned(srow, 4)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = y;
  a.K = K; a.N = N; a.M = VPQ_QMV_GROUPED_SLOTS; a.y_f32 = false; a.cu_count = g_dev.cu_count;
  a.gate_act = gate_act;
  if (bits == 8) {
    return finish(vpq::launch_qmv_rows8_sorted(reinterpret_cast<hipStream_t>(stream), a, tile2e, srow,
                                               npad / VPQ_QMV_GROUPED_SLOTS, n_experts));
  }
  return finish(vpq::launch_qmv_rows_sorted(reinterpret_cast<hipStream_t>(stream), a, tile2e, srow,
                                            npad / VPQ_QMV_GROUPED_SLOTS, x_from_srow, n_experts));
}

}  // namespace

int vpq_qmv_grouped_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int npad,
                                     const int32_t* tile2e, const int32_t* srow, int n_experts, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return sorted_qmv_common(stream, w, scales, biases, x, y, K, N, npad, tile2e, srow, n_experts, activation, true);
}

int vpq_qmv_grouped_down_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int npad,
                                    const int32_t* tile2e, const int32_t* srow, int n_experts)
{
  return sorted_qmv_common(stream, w, scales, biases, x, y, K, N, npad, tile2e, srow, n_experts, 0, false);
}

int vpq_qmv_grouped_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int npad,
                                     const int32_t* tile2e, const int32_t* srow, int n_experts, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return sorted_qmv_common(stream, w, scales, biases, x, y, K, N, npad, tile2e, srow, n_experts, activation, true, 8);
}

int vpq_qmv_grouped_down_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int npad,
                                    const int32_t* tile2e, const int32_t* srow, int n_experts)
{
  return sorted_qmv_common(stream, w, scales, biases, x, y, K, N, npad, tile2e, srow, n_experts, 0, false, 8);
}

int vpq_sample_topp_bf16(vpq_stream_t stream, const uint16_t* logits, int32_t* out_id, int V, float temp,
                         float top_p, uint32_t seed, uint16_t* ws, int n_iter, float rep_penalty,
                         float presence_penalty, int top_k, float min_p, uint8_t* seen)
{
  if (logits == nullptr || out_id == nullptr || ws == nullptr || seen == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (V < 1 || n_iter < 0 || rep_penalty == 0.0f) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(logits, 2) || !aligned(ws, 2) || !aligned(out_id, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_sample_topp(reinterpret_cast<hipStream_t>(stream), logits, out_id, V, temp, top_p, seed, ws,
                                        n_iter, rep_penalty, presence_penalty, top_k, min_p, seen));
}

size_t vpq_sample_hist_workspace_bytes(int n_slabs)
{
  return n_slabs >= 1 && n_slabs <= 1024 ? vpq::sample_hist_work_words(n_slabs) * sizeof(float) : 0;
}

int vpq_sample_hist_bf16(vpq_stream_t stream, const uint16_t* logits, int32_t* out_id, int V, float temp,
                         float top_p, uint32_t seed, uint16_t* ws, float rep_penalty, float presence_penalty,
                         int top_k, float min_p, uint8_t* seen, int n_slabs, void* work, size_t work_bytes)
{
  if (logits == nullptr || out_id == nullptr || ws == nullptr || seen == nullptr) { return VPQ_ERR_NULL_POINTER; }
  // counts travel as fp32: exact up to 2^24 logits
  if (V < 1 || V > (1 << 24) || rep_penalty == 0.0f || n_slabs < 1 || n_slabs > 1024) { return VPQ_ERR_BAD_SHAPE; }
  // a slab's fixed-point mass of one bin stays below 2^32
  if (((long long)V + n_slabs - 1) / n_slabs > 65535) { return VPQ_ERR_BAD_SHAPE; }
  if (work == nullptr || work_bytes < vpq_sample_hist_workspace_bytes(n_slabs)) { return VPQ_ERR_WORKSPACE; }
  if (!aligned(logits, 2) || !aligned(ws, 2) || !aligned(out_id, 4) || !aligned(work, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_sample_hist(reinterpret_cast<hipStream_t>(stream), logits, out_id, V, temp, top_p, seed, ws,
                                        rep_penalty, presence_penalty, top_k, min_p, seen, n_slabs,
                                        static_cast<float*>(work)));
}

int vpq_qmm_grouped_block_rows(void) { return vpq::kGroupedBlockRows; }

size_t vpq_moe_sort_workspace_bytes(int n_experts)
{
  return n_experts > 0 ? (size_t)3 * (size_t)n_experts * sizeof(int32_t) : 0;
}

int vpq_moe_sort_pairs(vpq_stream_t stream, const int32_t* pair_eid, int npair, int top_k, int n_experts,
                       int block_rows, int max_tiles, int32_t* tile2e, int32_t* srow, int32_t* sdst,
                       int32_t* ntiles, void* ws, size_t ws_bytes)
{
  if (pair_eid == nullptr || tile2e == nullptr || srow == nullptr || sdst == nullptr || ntiles == nullptr ||
      ws == nullptr) {
    return VPQ_ERR_NULL_POINTER;
  }
  if (npair < 1 || top_k < 1 || n_experts < 1 || block_rows < 1 || max_tiles < 1) { return VPQ_ERR_BAD_SHAPE; }
  if (npair > (1 << 24) || n_experts > 65536) { return VPQ_ERR_BAD_SHAPE; }
  // every expert's share rounded up to whole blocks must fit
  const long long need = ((long long)npair + block_rows - 1) / block_rows + (n_experts < npair ? n_experts : npair);
  if ((long long)max_tiles < need || (long long)max_tiles * block_rows > 0x7fffffffLL) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(pair_eid, 4) || !aligned(tile2e, 4) || !aligned(srow, 4) || !aligned(sdst, 4) || !aligned(ntiles, 4) ||
      !aligned(ws, 4)) {
    return VPQ_ERR_MISALIGNED;
  }
  if (ws_bytes < vpq_moe_sort_workspace_bytes(n_experts)) { return VPQ_ERR_WORKSPACE; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_moe_sort(reinterpret_cast<hipStream_t>(stream), pair_eid, npair, top_k, n_experts,
                                     block_rows, max_tiles, tile2e, srow, sdst, ntiles, static_cast<int*>(ws)));
}

int vpq_moe_scatter_back_bf16(vpq_stream_t stream, const uint16_t* dsorted, const int32_t* sdst, uint16_t* partials,
                              int npad, int H, int npair)
{
  if (dsorted == nullptr || sdst == nullptr || partials == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (npad < 1 || H < 1 || npair < 1 || (long long)npad * (long long)H > 0x3fffffffffLL) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(dsorted, 2) || !aligned(partials, 2) || !aligned(sdst, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  const bool wide = (H % 8) == 0 && aligned(dsorted, 16) && aligned(partials, 16);
  return finish(vpq::launch_moe_scatter_back(reinterpret_cast<hipStream_t>(stream), dsorted, sdst, partials, npad, H, npair,
                                             wide));
}

namespace {

int grouped_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, uint16_t* y, int K, int N, int npad, const int32_t* tile2e,
                   const int32_t* srow, const int32_t* sdst, int n_experts, int rows, int gate_act, int bits = 4)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr || tile2e == nullptr || (srow == nullptr && sdst == nullptr)) {
    return VPQ_ERR_NULL_POINTER;
  }
  if (npad < vpq::kGroupedBlockRows || (npad % vpq::kGroupedBlockRows) != 0 || n_experts < 1 || rows < 1) {
    return VPQ_ERR_BAD_SHAPE;
  }
  if (gate_act != 0 && (N & 1) != 0) { return VPQ_ERR_BAD_SHAPE; }
  // the kernel addresses rows of x by 32-bit byte offsets
  const long long xrows = srow != nullptr ? rows : npad;
  if (xrows * (long long)K * 2 >= 4000000000LL) { return VPQ_ERR_BAD_SHAPE; }
  // y rows are stored in 4- and 8-byte pieces
  if (!aligned(x, 16) || !aligned(y, 8) || !aligned(tile2e, 4) || (srow != nullptr && !aligned(srow, 4)) ||
      (sdst != nullptr && !aligned(sdst, 4))) {
    return VPQ_ERR_MISALIGNED;
  }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::GemmArgs g{};
  g.w = w; g.scales = scales; g.biases = biases; g.x = x; g.y = y;
  g.K = K; g.N = N; g.M = npad; g.lora_t = nullptr; g.lora_b = nullptr; g.r = 0;
  g.cu_count = g_dev.cu_count;
  g.gate_act = gate_act; g.out_stride = N / 2; g.out_off = 0;
  g.bits = bits;
  vpq::GroupedArgs ga{};
  ga.tile2e = tile2e; ga.srow = srow; ga.sdst = sdst;
  ga.n_experts = n_experts;
  ga.rows_x = srow != nullptr ? rows : npad;
  ga.rows_y = sdst != nullptr ? rows : npad;
  return finish(vpq::launch_qmm_grouped(reinterpret_cast<hipStream_t>(stream), g, ga));
}

}  // namespace

int vpq_qmm_grouped_gated_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                     int npad, const int32_t* tile2e, const int32_t* srow, int n_experts,
                                     int rows_x, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (srow == nullptr) { return VPQ_ERR_NULL_POINTER; }
  return grouped_common(stream, w, scales, biases, x, y, K, N, npad, tile2e, srow, nullptr, n_experts, rows_x,
                        activation);
}

int vpq_qmm_grouped_down_w4g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                    int npad, const int32_t* tile2e, const int32_t* sdst, int n_experts,
                                    int rows_y)
{
  if (sdst == nullptr) { return VPQ_ERR_NULL_POINTER; }
  return grouped_common(stream, w, scales, biases, x, y, K, N, npad, tile2e, nullptr, sdst, n_experts, rows_y, 0);
}

// ---- 8-bit twins on the fused kernels ----

namespace {

// The fused GEMM of a format twin (byte codes, groups of 32).  tile: 0 = by size, as for the 4-bit group-64 pack
// (the large-tile kernel once its tiles fill the CUs), 128 = the 256 x 128 tile kernel, 192 / 256 = the large-tile
// kernel at that width, -128 = the large-tile kernel at width 128.
int twin_gemm_launch(vpq_stream_t stream, const vpq::GemmArgs& g, int tile)
{
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (tile == 192 || tile == 256 || tile == -128) {
    // byte codes: up to 192 wide; groups of 32: 256 or 128 wide
    if (!vpq::qmm_big_supports(g) || (tile == 256 && g.bits == 8) || (tile == 192 && g.group == 32)) { return VPQ_ERR_BAD_SHAPE; }
    return finish(vpq::launch_qmm_big(hs, g, tile < 0 ? -tile : tile));
  }
  if (tile == 0 && vpq::qmm_big_supports(g)) {
    const int bn = vpq::qmm_big_tile_n(g.N, g.M, g_dev.cu_count, g.bits == 8 ? 192 : 256, g.group != 32);
    const long tiles = (long)((g.M + 255) / 256) * (long)((g.N + bn - 1) / bn);
    if (tiles >= (long)(g_dev.cu_count > 0 ? g_dev.cu_count : 256)) { return finish(vpq::launch_qmm_big(hs, g, bn)); }
  }
  return finish(vpq::launch_qmm_tile(hs, g));
}

}  // namespace

int vpq_qmm_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, uint16_t* y, int K, int N, int M, int out_stride, int out_off, int activation)
{
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (activation != 0 && activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (M <= 0 || out_off < 0 || (activation != 0 && (N & 1) != 0)) { return VPQ_ERR_BAD_SHAPE; }
  if (activation == 0 && (out_stride != 0 || out_off != 0)) { return VPQ_ERR_BAD_SHAPE; }
  if (out_stride > 0 && out_off + N / 2 > out_stride) { return VPQ_ERR_BAD_SHAPE; }
  if (out_stride <= 0 && out_off != 0) { return VPQ_ERR_BAD_SHAPE; }
  if ((long long)M * (long long)K * 2 >= 4000000000LL) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::GemmArgs g{};
  g.w = w; g.scales = scales; g.biases = biases; g.x = x; g.y = y;
  g.K = K; g.N = N; g.M = M; g.lora_t = nullptr; g.lora_b = nullptr; g.r = 0;
  g.cu_count = g_dev.cu_count;
  g.gate_act = activation; g.out_stride = out_stride; g.out_off = out_off;
  g.bits = 8;
  return twin_gemm_launch(stream, g, 0);
}

int vpq_qmm_tiled_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, uint16_t* y, int K, int N, int M, int activation, int tile_n)
{
  if (tile_n != 128 && tile_n != -128 && tile_n != 192) { return VPQ_ERR_BAD_SHAPE; }
  int st = check_pack(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (activation != 0 && activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (M <= 0 || (activation != 0 && (N & 1) != 0)) { return VPQ_ERR_BAD_SHAPE; }
  if ((long long)M * (long long)K * 2 >= 4000000000LL) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::GemmArgs g{};
  g.w = w; g.scales = scales; g.biases = biases; g.x = x; g.y = y;
  g.K = K; g.N = N; g.M = M;
  g.cu_count = g_dev.cu_count;
  g.gate_act = activation;
  g.bits = 8;
  return twin_gemm_launch(stream, g, tile_n);
}

int vpq_qmm_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       const uint16_t* x, uint16_t* y, int K, int N, int M)
{
  return vpq_qmm_gated_w8g64_bf16(stream, w, scales, biases, x, y, K, N, M, 0, 0, 0);
}

// Size-based entrances of the format twins (the ladder of vpq_linear_w4g64_bf16 without a workspace: slabs of
// the GEMV arithmetic up to 64 rows, the fused GEMM above).
int vpq_linear_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                          const uint16_t* x, uint16_t* y, int K, int N, int M)
{
  if (M >= 1 && M <= kSlabPlanMaxRows && x != nullptr && y != nullptr && K > 0 && N > 0) {
    for (int m0 = 0; m0 < M; m0 += 16) {
      const int rows = M - m0 < 16 ? M - m0 : 16;
      const int st = vpq_qmv_w8g64_bf16(stream, w, scales, biases, x + (size_t)m0 * K, y + (size_t)m0 * N, K, N, rows,
                                        nullptr);
      if (st != VPQ_OK) { return st; }
    }
    return VPQ_OK;
  }
  return vpq_qmm_w8g64_bf16(stream, w, scales, biases, x, y, K, N, M);
}

int vpq_qmm_grouped_gated_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                     int npad, const int32_t* tile2e, const int32_t* srow, int n_experts,
                                     int rows_x, int activation)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (srow == nullptr) { return VPQ_ERR_NULL_POINTER; }
  return grouped_common(stream, w, scales, biases, x, y, K, N, npad, tile2e, srow, nullptr, n_experts, rows_x,
                        activation, 8);
}

int vpq_qmm_grouped_down_w8g64_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                    const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N,
                                    int npad, const int32_t* tile2e, const int32_t* sdst, int n_experts,
                                    int rows_y)
{
  if (sdst == nullptr) { return VPQ_ERR_NULL_POINTER; }
  return grouped_common(stream, w, scales, biases, x, y, K, N, npad, tile2e, nullptr, sdst, n_experts, rows_y, 0, 8);
}


namespace {

int check_pack_g32(const uint32_t* w, const uint16_t* scales, const uint16_t* biases, int K, int N, bool scale_only)
{
  if (w == nullptr || scales == nullptr || (!scale_only && biases == nullptr)) { return VPQ_ERR_NULL_POINTER; }
  if (K <= 0 || N <= 0 || (K % 32) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(w, 16) || !aligned(scales, 2) || (!scale_only && !aligned(biases, 2))) { return VPQ_ERR_MISALIGNED; }
  return VPQ_OK;
}

int qmv_g32_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, void* y, bool y_f32, int K, int N, int M, const uint16_t* residual,
                   int gate_act, bool scale_only)
{
  int st = check_pack_g32(w, scales, biases, K, N, scale_only);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 16) { return VPQ_ERR_BAD_SHAPE; }
  const bool gelu_mul = gate_act == vpq::kStoreGeluMul;       // `residual` is the multiplier [N]
  if (gelu_mul && residual == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (gate_act != 0 && !gelu_mul && ((N & 1) != 0 || residual != nullptr)) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, y_f32 ? 4 : 2) || (residual != nullptr && !aligned(residual, 2))) {
    return VPQ_ERR_MISALIGNED;
  }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.w = w; a.scales = scales; a.biases = biases; a.x = x; a.y = y; a.residual = residual;
  a.K = K; a.N = N; a.M = M; a.y_f32 = y_f32; a.cu_count = g_dev.cu_count;
  a.gate_act = gate_act;
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (gelu_mul) { return finish(vpq::launch_qmv_simple_g32(hs, a, scale_only)); }    // the kernel that has this store
  // up to two rows of x: the row-streaming kernel; more: one wavefront per weight row
  if (M <= 2) { return finish(vpq::launch_qmv_rows_g32(hs, a, scale_only)); }
  return finish(vpq::launch_qmv_simple_g32(hs, a, scale_only));
}

}  // namespace

int vpq_dequant_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                           uint16_t* w_deq, int K, int N)
{
  int st = check_pack_g32(w, scales, biases, K, N, false);
  if (st != VPQ_OK) { return st; }
  if (w_deq == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (!aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_dequant_g32(reinterpret_cast<hipStream_t>(stream), w, scales, biases, w_deq, K, N));
}

int vpq_qmv_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       const uint16_t* x, uint16_t* y, int K, int N, int M, const uint16_t* residual, int scale_only)
{
  return qmv_g32_common(stream, w, scales, biases, x, y, false, K, N, M, residual, 0, scale_only != 0);
}

int vpq_qmv_w4g32_f32out(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                         const uint16_t* x, float* y, int K, int N, int M, int scale_only)
{
  return qmv_g32_common(stream, w, scales, biases, x, y, true, K, N, M, nullptr, 0, scale_only != 0);
}

int vpq_qmv_gelu_mul_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                                const uint16_t* x, uint16_t* y, int K, int N, const uint16_t* mul, int scale_only)
{
  return qmv_g32_common(stream, w, scales, biases, x, y, false, K, N, 1, mul, vpq::kStoreGeluMul, scale_only != 0);
}

int vpq_qmv_gated_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, uint16_t* y, int K, int N, int M, int activation, int scale_only)
{
  if (activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  return qmv_g32_common(stream, w, scales, biases, x, y, false, K, N, M, nullptr, activation, scale_only != 0);
}

namespace {

int qmm_g32_common(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   const uint16_t* x, uint16_t* y, int K, int N, int M, int activation, int tile_n)
{
  int st = check_pack_g32(w, scales, biases, K, N, false);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (activation != 0 && activation != VPQ_GATE_SWIGLU && activation != VPQ_GATE_GEGLU) { return VPQ_ERR_BAD_SHAPE; }
  if (M <= 0 || (K % 64) != 0 || (activation != 0 && (N & 1) != 0)) { return VPQ_ERR_BAD_SHAPE; }
  if ((long long)M * (long long)K * 2 >= 4000000000LL) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::GemmArgs g{};
  g.w = w; g.scales = scales; g.biases = biases; g.x = x; g.y = y;
  g.K = K; g.N = N; g.M = M; g.lora_t = nullptr; g.lora_b = nullptr; g.r = 0;
  g.cu_count = g_dev.cu_count;
  g.gate_act = activation; g.out_stride = 0; g.out_off = 0;
  g.group = 32;
  return twin_gemm_launch(stream, g, tile_n);
}

}  // namespace

int vpq_qmm_gated_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, uint16_t* y, int K, int N, int M, int activation)
{
  return qmm_g32_common(stream, w, scales, biases, x, y, K, N, M, activation, 0);
}

int vpq_qmm_tiled_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, uint16_t* y, int K, int N, int M, int activation, int tile_n)
{
  if (tile_n != 128 && tile_n != -128 && tile_n != 192 && tile_n != 256) { return VPQ_ERR_BAD_SHAPE; }
  return qmm_g32_common(stream, w, scales, biases, x, y, K, N, M, activation, tile_n);
}

int vpq_qmm_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       const uint16_t* x, uint16_t* y, int K, int N, int M)
{
  return vpq_qmm_gated_w4g32_bf16(stream, w, scales, biases, x, y, K, N, M, 0);
}

int vpq_linear_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                          const uint16_t* x, uint16_t* y, int K, int N, int M)
{
  // K % 64 != 0 (a group-32 pack may have K % 64 == 32) has no fused GEMM: slabs at every M
  if (M >= 1 && (M <= kSlabPlanMaxRows || (K % 64) != 0) && x != nullptr && y != nullptr && K > 0 && N > 0) {
    for (int m0 = 0; m0 < M; m0 += 16) {
      const int rows = M - m0 < 16 ? M - m0 : 16;
      const int st = vpq_qmv_w4g32_bf16(stream, w, scales, biases, x + (size_t)m0 * K, y + (size_t)m0 * N, K, N, rows,
                                        nullptr, 0);
      if (st != VPQ_OK) { return st; }
    }
    return VPQ_OK;
  }
  return vpq_qmm_w4g32_bf16(stream, w, scales, biases, x, y, K, N, M);
}

int vpq_qmm_dense_route_w4g32_bf16(vpq_stream_t stream, const uint32_t* w, const uint16_t* scales,
                                   const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                   uint16_t* w_deq, int expand)
{
  int st = check_pack_g32(w, scales, biases, K, N, false);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (w_deq == nullptr) { return VPQ_ERR_WORKSPACE; }
  if (M <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16) || !aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (expand != 0) {
    st = finish(vpq::launch_dequant_g32(hs, w, scales, biases, w_deq, K, N));
    if (st != VPQ_OK) { return st; }
  }
  std::string why;
  const int rc = vpq::dense_gemm_bf16(hs, x, w_deq, y, M, N, K, g_dev.cu_count, &why);
  if (rc != 0) {
    strncpy(g_last_error, why.c_str(), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return VPQ_ERR_DEVICE;
  }
  return VPQ_OK;
}

size_t vpq_argmax_workspace_bytes(int V, int rows)
{
  if (V <= 0 || rows <= 0) { return 0; }
  return (size_t)rows * (size_t)vpq::argmax_parts(V) * 2 * sizeof(float);
}

int vpq_argmax_bf16(vpq_stream_t stream, const uint16_t* logits, int32_t* out_id, int V, int rows, void* ws,
                    size_t ws_bytes)
{
  if (logits == nullptr || out_id == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (V <= 0 || rows <= 0 || rows > 65535) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(logits, 2) || !aligned(out_id, 4) || (ws != nullptr && !aligned(ws, 4))) { return VPQ_ERR_MISALIGNED; }
  if (ws != nullptr && ws_bytes < vpq_argmax_workspace_bytes(V, rows)) { return VPQ_ERR_WORKSPACE; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (ws == nullptr) { return finish(vpq::launch_argmax_row(hs, logits, out_id, V, rows)); }
  const int parts = vpq::argmax_parts(V);
  const int e = finish(vpq::launch_argmax_partial(hs, logits, static_cast<float*>(ws), V, rows, parts));
  if (e != VPQ_OK) { return e; }
  return finish(vpq::launch_argmax_combine(hs, static_cast<const float*>(ws), out_id, rows, parts));
}

int vpq_argmax_bf16_static(vpq_stream_t stream, const uint16_t* logits, int32_t* out_id, int V, int rows)
{
  if (logits == nullptr || out_id == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (V <= 0 || rows <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (rows > vpq::kArgmaxStaticRows) {
    snprintf(g_last_error, sizeof(g_last_error), "vpq_argmax_bf16_static: %d rows, the static scratch holds %d", rows,
             vpq::kArgmaxStaticRows);
    return VPQ_ERR_WORKSPACE;
  }
  if (!aligned(logits, 2) || !aligned(out_id, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  float* partials = nullptr;
  const hipError_t se = vpq::argmax_static_scratch(&partials);
  if (se != hipSuccess) { return device_error(se); }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  // Every pair the combine reads is written by this call's first stage: nothing of an earlier call is read,
  // so nothing has to be cleared.
  const int parts = vpq::argmax_parts(V);
  const int e = finish(vpq::launch_argmax_partial(hs, logits, partials, V, rows, parts));
  if (e != VPQ_OK) { return e; }
  return finish(vpq::launch_argmax_combine(hs, partials, out_id, rows, parts));
}

int vpq_argmax_partial_bf16(vpq_stream_t stream, const uint16_t* logits, float* partials, int V, int parts)
{
  if (logits == nullptr || partials == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (V <= 0 || parts < 1 || parts > 65535) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(logits, 2) || !aligned(partials, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_argmax_partial(reinterpret_cast<hipStream_t>(stream), logits, partials, V, 1, parts));
}

int vpq_argmax_combine(vpq_stream_t stream, const float* partials, int32_t* out_id, int parts)
{
  if (partials == nullptr || out_id == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (parts < 1) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(partials, 4) || !aligned(out_id, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_argmax_combine(reinterpret_cast<hipStream_t>(stream), partials, out_id, 1, parts));
}

int vpq_qmv_group_w4g64_bf16(vpq_stream_t stream, int count, const uint32_t* const* w,
                             const uint16_t* const* scales, const uint16_t* const* biases,
                             const uint16_t* x, uint16_t* const* y, int K, const int* N, int M)
{
  if (w == nullptr || scales == nullptr || biases == nullptr || y == nullptr || N == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (count < 1 || count > 4) { return VPQ_ERR_BAD_SHAPE; }
  // The tile kernel's grouped form where its shapes allow, else the row-streaming kernel's (M <= 2).
  bool mfma_group = vpq::qmv_mfma_supports(K, 1, M);
  for (int i = 0; i < count; ++i) {
    int st = check_pack(w[i], scales[i], biases[i], K, N[i]);
    if (st != VPQ_OK) { return st; }
    if (y[i] == nullptr) { return VPQ_ERR_NULL_POINTER; }
    if (!aligned(y[i], 2)) { return VPQ_ERR_MISALIGNED; }
    mfma_group = mfma_group && aligned(scales[i], 16) && aligned(biases[i], 16);
  }
  if (x == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 16) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16)) { return VPQ_ERR_MISALIGNED; }
  if (!mfma_group && !vpq::qmv_rows_supports(K, 1, M)) {
    for (int i = 0; i < count; ++i) {
      const int st = vpq_qmv_w4g64_bf16(stream, w[i], scales[i], biases[i], x, y[i], K, N[i], M, nullptr, nullptr, 0,
                                        VPQ_QMV_AUTO);
      if (st != VPQ_OK) { return st; }
    }
    return VPQ_OK;
  }
  int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.x = x; a.K = K; a.M = M; a.y_f32 = false; a.cu_count = g_dev.cu_count;
  vpq::QmvGroup g;
  g.count = count;
  for (int i = 0; i < count; ++i) { g.seg[i] = vpq::QmvSeg{w[i], scales[i], biases[i], y[i], N[i]}; }
  if (mfma_group && vpq::qmv_flow_supports(K, 1, M)) {
    return finish(vpq::launch_qmv_flow_group(reinterpret_cast<hipStream_t>(stream), a, g));
  }
  if (!mfma_group) { return finish(vpq::launch_qmv_rows_group(reinterpret_cast<hipStream_t>(stream), a, g)); }
  return finish(vpq::launch_qmv_mfma_group(reinterpret_cast<hipStream_t>(stream), a, g));
}

// The fused-QKV GEMV of the format twins (`affine_qmv_qkv_w4g32`, `affine_qmv_qkv_w8g64`,
// gpu-kernels/metal/quant/affine_qmv.metal:518-559): 1..4 packs that share x.  Group-32 packs at up to two rows of x
// run as one launch of the row-streaming kernel; otherwise the packs are separate calls, with the same bits.
int vpq_qmv_group_w4g32_bf16(vpq_stream_t stream, int count, const uint32_t* const* w, const uint16_t* const* scales,
                             const uint16_t* const* biases, const uint16_t* x, uint16_t* const* y, int K, const int* N,
                             int M, int scale_only)
{
  if (w == nullptr || scales == nullptr || y == nullptr || N == nullptr || (biases == nullptr && scale_only == 0)) {
    return VPQ_ERR_NULL_POINTER;
  }
  if (count < 1 || count > 4) { return VPQ_ERR_BAD_SHAPE; }
  if (x == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 16) { return VPQ_ERR_BAD_SHAPE; }
  for (int i = 0; i < count; ++i) {
    const int st = check_pack_g32(w[i], scales[i], scale_only ? nullptr : biases[i], K, N[i], scale_only != 0);
    if (st != VPQ_OK) { return st; }
    if (y[i] == nullptr) { return VPQ_ERR_NULL_POINTER; }
    if (!aligned(y[i], 2)) { return VPQ_ERR_MISALIGNED; }
  }
  if (!aligned(x, 16)) { return VPQ_ERR_MISALIGNED; }
  if (M > 2) {
    for (int i = 0; i < count; ++i) {
      const int st = vpq_qmv_w4g32_bf16(stream, w[i], scales[i], scale_only ? nullptr : biases[i], x, y[i], K, N[i], M,
                                        nullptr, scale_only);
      if (st != VPQ_OK) { return st; }
    }
    return VPQ_OK;
  }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.x = x; a.K = K; a.M = M; a.y_f32 = false; a.cu_count = g_dev.cu_count;
  vpq::QmvGroup g;
  g.count = count;
  for (int i = 0; i < count; ++i) { g.seg[i] = vpq::QmvSeg{w[i], scales[i], scale_only ? nullptr : biases[i], y[i], N[i]}; }
  return finish(vpq::launch_qmv_rows_group(reinterpret_cast<hipStream_t>(stream), a, g, 32, scale_only != 0));
}

int vpq_qmv_group_w8g64_bf16(vpq_stream_t stream, int count, const uint32_t* const* w, const uint16_t* const* scales,
                             const uint16_t* const* biases, const uint16_t* x, uint16_t* const* y, int K, const int* N,
                             int M)
{
  if (w == nullptr || scales == nullptr || biases == nullptr || y == nullptr || N == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (count < 1 || count > 4) { return VPQ_ERR_BAD_SHAPE; }
  for (int i = 0; i < count; ++i) {
    const int st = vpq_qmv_w8g64_bf16(stream, w[i], scales[i], biases[i], x, y[i], K, N[i], M, nullptr);
    if (st != VPQ_OK) { return st; }
  }
  return VPQ_OK;
}

int vpq_rmsnorm_bf16(vpq_stream_t stream, const uint16_t* x, const uint16_t* norm_w, uint16_t* out, int K, int M, float eps)
{
  if (x == nullptr || norm_w == nullptr || out == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (K < 1 || M < 1 || M > 65535 || !(eps >= 0.0f)) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 2) || !aligned(norm_w, 2) || !aligned(out, 2)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_rmsnorm(reinterpret_cast<hipStream_t>(stream), x, norm_w, out, K, M, eps));
}

// `affine_qmv_qkv_rms_w4g64` / `_w4g32` / `_w8g64` (gpu-kernels/metal/quant/affine_qmv.metal:671-740): RMSNorm of the
// one row of x, then the fused-QKV GEMV over the normalized row.  format: 0 = 4-bit group-64, 1 = 4-bit group-32,
// 2 = 8-bit group-64.  x_norm_ws: K elements of scratch that receive the normalized row.
int vpq_qmv_qkv_rms_bf16(vpq_stream_t stream, int format, int count, const uint32_t* const* w, const uint16_t* const* scales,
                         const uint16_t* const* biases, const uint16_t* x, const uint16_t* norm_w, uint16_t* const* y,
                         int K, const int* N, float eps, uint16_t* x_norm_ws)
{
  if (format < 0 || format > 2) { return VPQ_ERR_BAD_SHAPE; }
  if (x_norm_ws == nullptr) { return VPQ_ERR_WORKSPACE; }
  if (!aligned(x_norm_ws, 16)) { return VPQ_ERR_MISALIGNED; }
  // (the packs themselves are checked by the format's own grouped entry point below: a refusal there has written the
  // scratch and nothing else)
  if (w == nullptr || scales == nullptr || biases == nullptr || y == nullptr || N == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (count < 1 || count > 4) { return VPQ_ERR_BAD_SHAPE; }
  if (K <= 0 || (K % (format == 1 ? 32 : 64)) != 0) { return VPQ_ERR_BAD_SHAPE; }
  int st = vpq_rmsnorm_bf16(stream, x, norm_w, x_norm_ws, K, 1, eps);
  if (st != VPQ_OK) { return st; }
  if (format == 1) { return vpq_qmv_group_w4g32_bf16(stream, count, w, scales, biases, x_norm_ws, y, K, N, 1, 0); }
  if (format == 2) { return vpq_qmv_group_w8g64_bf16(stream, count, w, scales, biases, x_norm_ws, y, K, N, 1); }
  return vpq_qmv_group_w4g64_bf16(stream, count, w, scales, biases, x_norm_ws, y, K, N, 1);
}

int vpq_qmv_group_w4g64_f16(vpq_stream_t stream, int count, const uint32_t* const* w,
                            const uint16_t* const* scales, const uint16_t* const* biases,
                            const uint16_t* x, uint16_t* const* y, int K, const int* N, int M)
{
  if (w == nullptr || scales == nullptr || biases == nullptr || y == nullptr || N == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (count < 1 || count > 4) { return VPQ_ERR_BAD_SHAPE; }
  bool one_launch = vpq::qmv_flow_supports(K, 1, M);
  for (int i = 0; i < count; ++i) {
    int st = check_pack(w[i], scales[i], biases[i], K, N[i]);
    if (st != VPQ_OK) { return st; }
    if (y[i] == nullptr) { return VPQ_ERR_NULL_POINTER; }
    if (!aligned(y[i], 2)) { return VPQ_ERR_MISALIGNED; }
    one_launch = one_launch && aligned(scales[i], 16) && aligned(biases[i], 16);
  }
  if (x == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (M < 1 || M > 16) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16)) { return VPQ_ERR_MISALIGNED; }
  if (!one_launch) {
    for (int i = 0; i < count; ++i) {
      const int st = vpq_qmv_w4g64_f16(stream, w[i], scales[i], biases[i], x, y[i], K, N[i], M, nullptr);
      if (st != VPQ_OK) { return st; }
    }
    return VPQ_OK;
  }
  int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  vpq::QmvArgs a{};
  a.x = x; a.K = K; a.M = M; a.y_f32 = false; a.cu_count = g_dev.cu_count;
  vpq::QmvGroup g;
  g.count = count;
  for (int i = 0; i < count; ++i) { g.seg[i] = vpq::QmvSeg{w[i], scales[i], biases[i], y[i], N[i]}; }
  return finish(vpq::launch_qmv_flow_group(reinterpret_cast<hipStream_t>(stream), a, g, true));
}

int vpq_quantize_w4g64(vpq_stream_t stream, const uint16_t* src, uint32_t* w, uint16_t* scales_f16,
                       uint16_t* biases_f16, int K, int N, float clip)
{
  if (src == nullptr || w == nullptr || scales_f16 == nullptr || biases_f16 == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (K <= 0 || N <= 0 || (K % 64) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(src, 16) || !aligned(w, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_quantize(reinterpret_cast<hipStream_t>(stream), src, w, scales_f16, biases_f16, K, N, clip));
}

int vpq_quantize(vpq_stream_t stream, int bits, int group, int src_f16, const uint16_t* src, uint32_t* w,
                 uint16_t* scales_f16, uint16_t* biases_f16, int K, int N, float clip)
{
  if (src == nullptr || w == nullptr || scales_f16 == nullptr || biases_f16 == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if ((bits != 4 && bits != 8) || (group != 64 && group != 32)) { return VPQ_ERR_BAD_SHAPE; }
  if (K <= 0 || N <= 0 || (K % group) != 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(src, 16) || !aligned(w, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_quantize(reinterpret_cast<hipStream_t>(stream), src, w, scales_f16, biases_f16, K, N, clip, bits,
                                     group, src_f16 != 0));
}

int vpq_f16_to_bf16(vpq_stream_t stream, const uint16_t* in_f16, uint16_t* out_bf16, size_t count)
{
  if (in_f16 == nullptr || out_bf16 == nullptr) { return VPQ_ERR_NULL_POINTER; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_f16_to_bf16(reinterpret_cast<hipStream_t>(stream), in_f16, out_bf16, count));
}

int vpq_profile_empty_kernel(vpq_stream_t stream, void* sink)
{
  if (sink == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (!aligned(sink, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_profile_empty(reinterpret_cast<hipStream_t>(stream), static_cast<uint32_t*>(sink)));
}

int vpq_profile_read_kernel(vpq_stream_t stream, const void* src, size_t bytes, void* sink)
{
  if (src == nullptr || sink == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (bytes < 16) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(src, 16) || !aligned(sink, 4)) { return VPQ_ERR_MISALIGNED; }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_profile_read(reinterpret_cast<hipStream_t>(stream), src, bytes, static_cast<uint32_t*>(sink)));
}

int vpq_profile_enable(int max_launches)
{
  vpq::ProfileState& ps = vpq::profile_state();
  if (max_launches <= 0) {
    ps.on = false;
    return VPQ_OK;
  }
  const int st = ensure_init();
  if (st != VPQ_OK) { return st; }
  while (ps.events.size() < (size_t)max_launches * 2) {
    hipEvent_t e;
    const hipError_t err = hipEventCreate(&e);
    if (err != hipSuccess) { return device_error(err); }
    ps.events.push_back(e);
  }
  ps.used = 0;
  ps.on = true;
  return VPQ_OK;
}

int vpq_profile_read(float* kernel_ms, int capacity)
{
  vpq::ProfileState& ps = vpq::profile_state();
  const int n = (int)(ps.used / 2);
  for (int i = 0; i < n && i < capacity; ++i) {
    hipError_t err = hipEventSynchronize(ps.events[2 * i + 1]);
    if (err != hipSuccess) { return device_error(err); }
    float ms = 0.0f;
    err = hipEventElapsedTime(&ms, ps.events[2 * i], ps.events[2 * i + 1]);
    if (err != hipSuccess) { return device_error(err); }
    if (kernel_ms != nullptr) { kernel_ms[i] = ms; }
  }
  ps.used = 0;
  return n;
}

// 8-bit codes on IEEE binary16 elements (the half build's affine_dequant_w8g64 / _w8g32 and affine_qmm_steel_w8g64 /
// _w8g32): the expansion, and the GEMM by the dequant-once route on the binary16 dense GEMM.
int vpq_dequant_w8_f16(vpq_stream_t stream, int group, const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                       uint16_t* w_deq, int K, int N)
{
  if (group != 64 && group != 32) { return VPQ_ERR_BAD_SHAPE; }
  int st = group == 64 ? check_pack(w, scales, biases, K, N) : check_pack_w8g32(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (w_deq == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (!aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  return finish(vpq::launch_dequant8(reinterpret_cast<hipStream_t>(stream), w, scales, biases, w_deq, K, N, group, true));
}

int vpq_qmm_dense_route_w8_f16(vpq_stream_t stream, int group, const uint32_t* w, const uint16_t* scales,
                               const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                               uint16_t* w_deq, int expand)
{
  if (group != 64 && group != 32) { return VPQ_ERR_BAD_SHAPE; }
  int st = group == 64 ? check_pack(w, scales, biases, K, N) : check_pack_w8g32(w, scales, biases, K, N);
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (w_deq == nullptr) { return VPQ_ERR_WORKSPACE; }
  if (M <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16) || !aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (expand != 0) {
    st = finish(vpq::launch_dequant8(hs, w, scales, biases, w_deq, K, N, group, true));
    if (st != VPQ_OK) { return st; }
  }
  std::string why;
  const int rc = vpq::dense_gemm_elt(hs, x, w_deq, y, M, N, K, true, g_dev.cu_count, &why);
  if (rc != 0) {
    strncpy(g_last_error, why.c_str(), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return VPQ_ERR_DEVICE;
  }
  return VPQ_OK;
}

// The dequant-once route with the runtime adapter for any of the pack formats: the adapter's pre-pass, the format's
// expansion (or the kept one), the dense GEMM with t . B^T in the same accumulators.
int vpq_qmm_dense_route_lora_bf16(vpq_stream_t stream, int format, const uint32_t* w, const uint16_t* scales,
                                  const uint16_t* biases, const uint16_t* x, uint16_t* y, int K, int N, int M,
                                  uint16_t* w_deq, int expand, const uint16_t* lora_a, const uint16_t* lora_b, int r,
                                  float alpha, uint16_t* lora_t_ws)
{
  if (format == VPQ_FORMAT_W4G64) {
    return vpq_qmm_dense_route_lora_w4g64_bf16(stream, w, scales, biases, x, y, K, N, M, w_deq, expand, lora_a, lora_b, r,
                                               alpha, lora_t_ws);
  }
  int st = format == VPQ_FORMAT_W4G32   ? check_pack_g32(w, scales, biases, K, N, false)
           : format == VPQ_FORMAT_W8G64 ? check_pack(w, scales, biases, K, N)
           : format == VPQ_FORMAT_W8G32 ? check_pack_w8g32(w, scales, biases, K, N)
                                        : VPQ_ERR_BAD_SHAPE;
  if (st != VPQ_OK) { return st; }
  if (x == nullptr || y == nullptr) { return VPQ_ERR_NULL_POINTER; }
  if (w_deq == nullptr) { return VPQ_ERR_WORKSPACE; }
  if (M <= 0) { return VPQ_ERR_BAD_SHAPE; }
  if (!aligned(x, 16) || !aligned(y, 16) || !aligned(w_deq, 16)) { return VPQ_ERR_MISALIGNED; }
  const bool lora = lora_a != nullptr && alpha != 0.0f;
  if (lora) {
    if (lora_b == nullptr) { return VPQ_ERR_NULL_POINTER; }
    if (lora_t_ws == nullptr) { return VPQ_ERR_WORKSPACE; }
    // the pre-pass walks K in chunks of 64
    if (r < 8 || r > vpq::kLoraMaxRank || (r % 8) != 0 || (K % 64) != 0) { return VPQ_ERR_BAD_SHAPE; }
    if (!aligned(lora_a, 16) || !aligned(lora_b, 16) || !aligned(lora_t_ws, 16)) { return VPQ_ERR_MISALIGNED; }
  }
  st = ensure_init();
  if (st != VPQ_OK) { return st; }
  hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
  if (lora) {
    st = finish(vpq::launch_lora_a(hs, x, lora_a, lora_t_ws, M, K, r, alpha));
    if (st != VPQ_OK) { return st; }
  }
  if (expand != 0) {
    st = finish(format == VPQ_FORMAT_W4G32   ? vpq::launch_dequant_g32(hs, w, scales, biases, w_deq, K, N)
                : format == VPQ_FORMAT_W8G64 ? vpq::launch_dequant8(hs, w, scales, biases, w_deq, K, N)
                                             : vpq::launch_dequant8(hs, w, scales, biases, w_deq, K, N, 32));
    if (st != VPQ_OK) { return st; }
  }
  std::string why;
  const int rc = vpq::dense_gemm_elt(hs, x, w_deq, y, M, N, K, false, g_dev.cu_count, &why, lora ? lora_t_ws : nullptr,
                                     lora ? lora_b : nullptr, lora ? r : 0);
  if (rc != 0) {
    strncpy(g_last_error, why.c_str(), sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return VPQ_ERR_DEVICE;
  }
  return VPQ_OK;
}

size_t vpq_weight_bytes(int N, int K) { return (size_t)N * (size_t)(K * 4 / 32) * 4; }
size_t vpq_scale_bytes(int N, int K) { return (size_t)N * (size_t)(K / 64) * 2; }

}  // extern "C"

// C++ host side of the w4g64 quantized-linear path, above the C ABI of
// include/vpq.h.  It keeps the call protocol of the reference's compute
// backend, so that a quantized-linear call site reads the same on both:
//
//   lib = QuantLibrary::load("affine_qmv_bf16");                 apple-silicon/metal-compute/metal-compute.h:298-301
//   fn  = lib.function("affine_qmv_w4g64");
//   enc = stream.begin_compute();                                command-stream.h
//   enc.set_function(fn);
//   enc.set_buffer(0, codes); (1, scales); (2, qbias); (3, x, x_off); (4, y, y_off);   compute-encoder.h:82-83
//   enc.set_constant(5, K); (6, N); [(7, M)]                                           compute-encoder.h:113-119
//   enc.dispatch(threads_per_grid, threads_per_threadgroup);                           compute-encoder.h:188-189
//   fence = stream.commit();  fence.wait_ok(&reason);                                  command-stream.h:92-99
//
// Same conventions as the reference: no exceptions; default-constructed handles
// are empty and every call on them is a no-op; set_buffer ignores an empty
// buffer; a failed dispatch (bad shape, missing slot, device error) is
// recorded on the stream and reported by Fence::wait_ok.  A CommandStream and
// its encoder are single-threaded objects; work is stream-ordered.
//
// The launch dimensions of the reference are threads of an Apple GPU and have no
// meaning for the CDNA4 kernels, which choose their own grids.  dispatch() reads
// from them only what the reference's kernels read from their grid position:
// the number of x rows M of `affine_qmv_w4g64` (grid.x / 32,
// gpu-kernels/metal/quant/affine_qmv.metal:186-284).
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <type_traits>
#include <vector>

namespace vpipe_amd {

struct LaunchDims {
  unsigned x = 1;
  unsigned y = 1;
  unsigned z = 1;
};

// Move-only RAII handle of device memory (the role of SharedBuffer,
// apple-silicon/metal-compute/shared-buffer.h:33-57).  wrap() makes a
// non-owning view of memory allocated elsewhere (a torch tensor, a checkpoint arena).
class DeviceBuffer {
public:
  DeviceBuffer() noexcept = default;
  DeviceBuffer(DeviceBuffer&& o) noexcept;
  DeviceBuffer& operator=(DeviceBuffer&& o) noexcept;
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  ~DeviceBuffer();

  static DeviceBuffer allocate(std::size_t bytes);             // empty on failure
  static DeviceBuffer wrap(void* device_ptr, std::size_t bytes) noexcept;

  bool empty() const noexcept { return _ptr == nullptr; }
  void* data() const noexcept { return _ptr; }
  std::size_t size() const noexcept { return _bytes; }
  bool upload(const void* host, std::size_t bytes, std::size_t byte_offset = 0) const;    // synchronous
  bool download(void* host, std::size_t bytes, std::size_t byte_offset = 0) const;        // synchronous

private:
  void* _ptr = nullptr;
  std::size_t _bytes = 0;
  bool _owned = false;
};

// Which C-ABI entry a function name of the reference's metallibs maps to.
enum class QuantKernel : std::uint8_t {
  None = 0,
  Dequant,        // affine_dequant_w4g64
  Qmv,            // affine_qmv_w4g64              M from grid.x / 32
  QmvAdd,         // affine_qmv_w4g64_add          slot 7 = residual buffer
  QmvBatch,       // affine_qmv_batch*_w4g64       slot 7 = m_total
  QmvBatchSwiglu, // affine_qmv_batch*_swiglu_w4g64: the gated GEMV over m_total rows (slot 7), N = 2 * ffn
  QmvBatchGeglu,  // affine_qmv_batch_geglu_w4g64 / _w4g32
  Qmm,            // affine_qmm_steel_w4g64[_bm64|_bm128], affine_qmm_mma_w4g64    slot 7 = M
  QmvQkv,         // affine_qmv_qkv_w4g64: row-concatenated q|k|v pack, slots 4,5,6 = q,k,v outputs,
                  //   7 = K, 8,9,10 = q_rows, k_rows, v_rows (v_rows == 0: q|k only); one launch
  QmvSwiglu,      // affine_qmv_swiglu_w4g64: interleaved gate|up pack, N = 2*ffn, y [M, ffn]; M from grid.x / 32
  QmmSwiglu,      // affine_qmm_swiglu_w4g64[_bm64|_bm128|_bm64_rs]: slot 7 = M, 8 = out_stride, 9 = out_off (_rs)
  QmvGeglu,       // affine_qmv_geglu_w4g64: as QmvSwiglu with gelu_tanh(gate) * up
  Requant84,      // affine_requant_w8_to_w4_g64: 0:w8 1:s8 2:b8 3:w4 4:s4 5:b4 6:K 7:N
  QuantizeBf16,   // affine_quant_w{4,8}_g{64,32} of the bf16 library: 0:x 1:w 2:scales(F16) 3:biases(F16) 4:K 5:N 6:clip (float)
  QuantizeF16,    // ... of the binary16 library (the source matrix is binary16)
  QmvGeluMul,     // affine_qmv_gelu_mul_w4g64: one row of x, slot 7 = mul buffer [N]; y = gelu_tanh(W x) * mul
  QmvQkvRms,      // affine_qmv_qkv_rms_w4g64 / _w4g32 / _w8g64: slots 0:w 1:scales 2:biases 3:x 4:norm_w 5:q 6:k 7:v 8:K
                  //   9,10,11 = q_rows, k_rows, v_rows, 12 = eps (float); the normalized row goes through stream scratch
  MoeGate,        // affine_moe_gate_w8g64: slots 0:w 1:scales 2:biases 3:x 4:gate 5:K; rows of x = grid.y
  QmmGeglu,       // affine_qmm_geglu_w4g64: as QmmSwiglu
  EmbedGather,    // dequant_embed_gather_f16: slots 0:ids 1:w 2:scales 3:biases 4:out 5:H; T = grid.y,
                  //   the vocabulary size is what the bound code buffer holds
  GatherSwiglu,   // affine_gather_qmv_swiglu_w4g64: expert batch [E, 2*inner, ...], slot 7 = pair_eid buffer,
                  //   8 = top_k; pairs = grid.z; the expert count is what the bound code buffer holds
  GatherGeglu,    // affine_gather_qmv_geglu_w4g64: as GatherSwiglu
  GatherDown,     // affine_gather_down_qmv_w4g64: x [npair, K], slot 7 = pair_eid buffer; pairs = grid.z
  GroupedSwiglu,  // affine_qmm_grouped_swiglu_w4g64: expert batch, x = hidden rows gathered through slot 9 = srow,
                  //   slot 7 = npad, 8 = tile2e; y [npad, N/2] in slot order
  GroupedGeglu,   // affine_qmm_grouped_geglu_w4g64: as GroupedSwiglu
  GroupedDown,    // affine_qmm_grouped_w4g64: x [npad, K] in slot order, slot 9 = sdst, y rows in pair order
  SortedSwiglu,   // affine_grouped_swiglu_w4g64: expert batch, tiles of two sorted slots (tile = grid.z), slot 7 = srow
                  //   (x row per slot, < 0 padding), 8 = tile2e; y [npad, N/2] in slot order
  SortedDown,     // affine_grouped_down_w4g64: x [npad, K] and y [npad, N] in slot order, slots 7, 8 as SortedSwiglu
  GatherSplit48,  // affine_gather_qmv_swiglu_w4w8g64: slots 0..2 gate pack (4-bit), 3..5 up pack (8-bit), 6:x 7:y 8:K
                  //   9:ffn 10:pair_eid 11:top_k; pairs = grid.z
  GatherSplit84,  // affine_gather_qmv_swiglu_w8w4g64: gate 8-bit, up 4-bit
  Argmax,         // argmax_f16: slots 0:logits 1:out_id 2:V (one workgroup)
  ArgmaxPartial,  // argmax_partial_f16: slots 0:logits 1:partials 2:V 3:M slabs
  ArgmaxCombine,  // argmax_combine_f16: slots 0:partials 1:out_id 2:M
  SampleTopp,     // sample_topp_f16: slots 0:logits 1:out_id 2:V 3:temp 4:top_p 5:seed 6:ws 7:n_iter 8:rep 9:pres
                  //   10:top_k 11:min_p 12:seen (one workgroup); float constants are 4-byte constants
};

// The packed format a function name ends in.
enum class QuantFormat : std::uint8_t {
  W4G64 = 0,      // _w4g64: 4-bit codes, a scale and a bias per 64 values
  W8G64,          // _w8g64: one byte per value
  W4G32,          // _w4g32: 4-bit codes, a scale and a bias per 32 values
  W4G32Q40,       // _w4g32_q40 / _w4g32_add_q40: as W4G32 with the bias buffer never read (bias = -8 * scale)
  W8G32,          // _w8g32: one byte per value, a scale and a bias per 32 values
  W4G64F16,       // the metallibs without the `_bf16` suffix ("affine_qmv", "affine_dequant"): IEEE binary16 elements
  W8G64F16,       // ... their 8-bit functions (expansion and GEMM)
  W8G32F16,
};

class QuantFunction {
public:
  QuantFunction() noexcept = default;
  bool valid() const noexcept { return _kind != QuantKernel::None; }
  QuantKernel kind() const noexcept { return _kind; }
  QuantFormat format() const noexcept { return _format; }
  const std::string& name() const noexcept { return _name; }

private:
  friend class QuantLibrary;
  QuantKernel _kind = QuantKernel::None;
  QuantFormat _format = QuantFormat::W4G64;
  std::string _name;
};

// The reference groups its kernels in metallibs loaded by name; the bf16 twins
// are the ones this path implements ("affine_qmv_bf16", "affine_qmm_steel_bf16",
// "affine_qmm_mma_bf16", "affine_dequant_bf16", and "llm_elementwise_bf16" for the dequantizing
// embedding gather).  Any other name gives an empty library.
class QuantLibrary {
public:
  QuantLibrary() noexcept = default;
  static QuantLibrary load(const std::string& name);
  bool valid() const noexcept { return !_name.empty(); }
  QuantFunction function(const std::string& fn_name) const;    // invalid if the library does not hold it

private:
  std::string _name;
};

class CommandStream;

class Fence {
public:
  Fence() noexcept = default;
  // Waits for everything committed before this fence.  False if a dispatch was rejected or the
  // device reported an error; *reason then says which.
  bool wait_ok(std::string* reason = nullptr);

private:
  friend class CommandStream;
  CommandStream* _stream = nullptr;
};

class ComputeEncoder {
public:
  ComputeEncoder() noexcept = default;
  ComputeEncoder(ComputeEncoder&& o) noexcept;
  ComputeEncoder& operator=(ComputeEncoder&& o) noexcept;
  ComputeEncoder(const ComputeEncoder&) = delete;
  ComputeEncoder& operator=(const ComputeEncoder&) = delete;
  ~ComputeEncoder();

  bool valid() const noexcept { return _stream != nullptr; }
  void set_function(const QuantFunction& fn);
  void set_buffer(unsigned index, const DeviceBuffer& buf, std::size_t byte_offset = 0);
  void set_constant_bytes(unsigned index, const void* bytes, std::size_t size);
  template <class T>
  void set_constant(unsigned index, const T& value)
  {
    static_assert(std::is_trivially_copyable<T>::value, "set_constant requires a trivially-copyable type");
    set_constant_bytes(index, &value, sizeof(T));
  }
  void dispatch(LaunchDims threads_per_grid, LaunchDims threads_per_threadgroup);

  // Dispatches inside the scope are independent of each other (unfused q|k|v, gate|up:
  // compute-encoder.h, ConcurrentScope): they go to side streams of the CommandStream
  // and run concurrently; leaving the scope joins them back into the main stream.
  class ConcurrentScope {
  public:
    ConcurrentScope(ConcurrentScope&& o) noexcept : _e(o._e) { o._e = nullptr; }
    ConcurrentScope& operator=(ConcurrentScope&&) = delete;
    ConcurrentScope(const ConcurrentScope&) = delete;
    ~ConcurrentScope();

  private:
    friend class ComputeEncoder;
    ConcurrentScope(ComputeEncoder* e, bool active) noexcept;
    ComputeEncoder* _e = nullptr;
  };
  ConcurrentScope concurrent_scope(bool active = true) { return ConcurrentScope(this, active); }

  void end();
  long dispatch_count() const noexcept { return _n_dispatch; }

private:
  friend class CommandStream;
  explicit ComputeEncoder(CommandStream* s) noexcept : _stream(s) {}
  static constexpr unsigned kSlots = 16;
  struct Slot {
    void* ptr = nullptr;
    std::size_t bytes = 0;       // bytes from ptr to the end of the bound buffer
    bool is_buffer = false;
    bool is_const = false;
    std::int64_t ivalue = 0;
    float fvalue = 0.f;
  };
  CommandStream* _stream = nullptr;
  QuantFunction _fn;
  Slot _slots[kSlots];
  long _n_dispatch = 0;
  int _scope_depth = 0;
  int _scope_next = 0;     // next side stream inside a concurrent scope
  int _scope_used = 0;     // side streams used by the current scope
};

// One HIP stream (plus side streams for concurrent scopes), the role of the
// reference's CommandStream (one Metal queue).  Errors of dispatches are kept
// here until a Fence is waited on.
class CommandStream {
public:
  CommandStream() noexcept = default;
  CommandStream(CommandStream&& o) noexcept;
  CommandStream& operator=(CommandStream&& o) noexcept;
  CommandStream(const CommandStream&) = delete;
  CommandStream& operator=(const CommandStream&) = delete;
  ~CommandStream();

  static CommandStream create();                        // new stream on the current device; empty on failure
  static CommandStream adopt(void* hip_stream);         // run on a stream owned by the caller
  bool valid() const noexcept { return _valid; }
  void* native() const noexcept { return _main; }       // hipStream_t
  ComputeEncoder begin_compute() { return valid() ? ComputeEncoder(this) : ComputeEncoder(); }
  Fence commit();
  // Split-K scratch handed to QMV dispatches; grown on demand between dispatches (the only
  // allocation this layer makes, like the reference's host-owned grow-once scratch,
  // generative-models/minimax-h3/metal-minimax-h3-transformer.cc:2049-2053).
  void* qmv_workspace(std::size_t bytes);
  void record_error(int status, const std::string& what);
  bool ok() const noexcept { return _error.empty(); }

private:
  friend class ComputeEncoder;
  friend class Fence;
  static constexpr int kSideStreams = 3;
  bool ensure_side_streams();
  void release();
  void* _main = nullptr;
  bool _owns_main = false;
  bool _valid = false;
  void* _side[kSideStreams] = {nullptr, nullptr, nullptr};
  void* _fork_event = nullptr;
  void* _join_event[kSideStreams] = {nullptr, nullptr, nullptr};
  DeviceBuffer _ws;
  std::string _error;
};

// The codes/scales/qbias triple of one Linear (generative-models/minimax-h3/
// metal-minimax-h3-transformer.h:596-608) and the optional runtime LoRA factors
// (:923-931: a[rank,K], b[N,rank]).  Offsets are byte offsets into the buffers.
struct Linear {
  const DeviceBuffer* codes = nullptr;
  const DeviceBuffer* scales = nullptr;
  const DeviceBuffer* qbias = nullptr;
  std::size_t codes_off = 0, scales_off = 0, qbias_off = 0;
  int K = 0, N = 0;
  int bits = 4, group = 64;          // (4, 64), (8, 64), (4, 32) or (8, 32): the pack formats the library serves
};

struct LoraFactors {
  const DeviceBuffer* a = nullptr;   // [rank, K] bf16
  const DeviceBuffer* b = nullptr;   // [N, rank] bf16
  int rank = 0;
  float strength = 1.0f;             // request strength applied at run time (.h:295-303)
};

// y[M,N] = x[M,K] . W^T (+ LoRA), choosing QMV or QMM by M like the reference's qmm_auto_
// (generative-models/qwen3/metal-qwen-model.cc:3964-4033).  `lora_t` is [M,rank] bf16 scratch.
void quant_linear_forward(CommandStream& stream, const Linear& lin, const DeviceBuffer& x, std::size_t x_off,
                          const DeviceBuffer& y, std::size_t y_off, int M, const LoraFactors* lora = nullptr,
                          const DeviceBuffer* lora_t = nullptr);

}  // namespace vpipe_amd

// On-disk side of the w4g64 path: the safetensors container the reference's quantizer writes
// and its model loaders read,
//     [u64 LE header_len][JSON header, space-padded][data blob]
// with, per quantized Linear `<prefix>`, `<prefix>.weight` U32 [N, K/8], `<prefix>.scales` F16
// [N, K/64] and `<prefix>.biases` F16 [N, K/64]
// (generative-models/quantize/safetensors-writer.h:10-39,
//  generative-models/llama3/metal-llama-weights.h:36-60).
//
//   PackFile    reader: one file or a sharded model directory merged into one namespace; the role
//               of MetalLlamaWeights (open / open_model / has / info / tensor_names / alignment).
//               The reference memory-maps a shard and copies a tensor into unified memory; a
//               discrete GPU has no use for the mapping, so tensors are read with pread(2) into
//               a host staging buffer and uploaded, and scales / biases are converted F16 -> bf16
//               on the device once, as a bf16 model does at load (docs/PLUGINS.md:210-213).
//   PackWriter  streaming writer: the role of SafetensorsWriter (add / close, shards by a byte
//               budget, data section and every 16-byte-multiple tensor on a 16-byte boundary,
//               model.safetensors.index.json).
//
// No exceptions: failures are empty optionals / false, with a reason where one helps.
#pragma once

#include <cstddef>
#include <cstdint>
#include <optional>
#include <string>
#include <unordered_map>
#include <vector>

#include "vpq_host.h"

namespace vpipe_amd {

struct TensorInfo {
  std::string dtype;                 // "U32", "F16", "BF16", "F32", ...
  std::vector<std::int64_t> shape;
  std::uint64_t offset = 0;          // bytes from the start of the shard's data blob
  std::uint64_t nbytes = 0;
  int shard = 0;
};

// One quantized Linear resident on the device, scales and zero points already bf16.
struct LoadedLinear {
  DeviceBuffer codes, scales, qbias;
  int K = 0, N = 0;
  int bits = 4, group = 64;
  Linear view() const
  {
    Linear l;
    l.codes = &codes; l.scales = &scales; l.qbias = &qbias;
    l.K = K; l.N = N;
    l.bits = bits; l.group = group;
    return l;
  }
};

class PackFile {
public:
  // A single named file.  nullopt on any error (unreadable, truncated, malformed header, a byte
  // range outside the file or disagreeing with dtype x shape).
  static std::optional<PackFile> open(const std::string& path, std::string* why = nullptr);
  // A model directory: model.safetensors.index.json (every shard it names, merged) or
  // model.safetensors.
  static std::optional<PackFile> open_model(const std::string& dir, std::string* why = nullptr);

  PackFile(PackFile&& o) noexcept;
  PackFile& operator=(PackFile&& o) noexcept;
  PackFile(const PackFile&) = delete;
  PackFile& operator=(const PackFile&) = delete;
  ~PackFile();

  bool has(const std::string& name) const { return _tensors.count(name) != 0; }
  const TensorInfo* info(const std::string& name) const;
  std::vector<std::string> tensor_names() const;
  int shard_count() const { return static_cast<int>(_shards.size()); }

  // How much of the checkpoint sits on 16-byte file offsets
  // (generative-models/llama3/metal-llama-weights.h:75-92).
  struct Alignment {
    std::size_t tensors = 0;
    std::size_t misaligned = 0;
    int shards = 0;
    int bad_shards = 0;              // shards whose data section itself is off
  };
  Alignment alignment() const;

  // Raw bytes of one tensor into memory the caller owns; false if absent, too small or short read.
  bool read_into(const std::string& name, void* dst, std::size_t capacity) const;

  // Bit width / group size of an affine Linear from its shapes and its input width K
  // (generative-models/qwen3/metal-qwen-model.cc:653-676): weight is [.., N, K*bits/32], scales
  // [.., N, K/group].  0 if the tensors are missing.
  int affine_bits(const std::string& prefix, int K) const;
  int affine_group(const std::string& prefix, int K) const;

  // Reads `<prefix>.weight/.scales/.biases`, checks that they are a 4-bit group-64 pack of input
  // width K (K == 0: taken from the weight shape), uploads them and converts F16 scales / biases
  // to bf16 on `stream`.  Synchronous.  False with *why on any mismatch.
  bool load_linear(CommandStream& stream, const std::string& prefix, int K, LoadedLinear* out,
                   std::string* why = nullptr) const;

private:
  PackFile() = default;
  struct Shard {
    std::string path;
    int fd = -1;
    std::uint64_t data_start = 0;
    std::uint64_t file_size = 0;
  };
  bool add_shard(const std::string& path, std::string* why);
  void release();
  std::vector<Shard> _shards;
  std::unordered_map<std::string, TensorInfo> _tensors;
};

class PackWriter {
public:
  explicit PackWriter(std::string out_dir, std::uint64_t shard_max_bytes = 5ull << 30);
  ~PackWriter();
  PackWriter(const PackWriter&) = delete;
  PackWriter& operator=(const PackWriter&) = delete;

  // Appends one tensor to the current shard; the bytes are written out before the call returns.
  // False on an IO error, a duplicate name or after close().
  bool add(const std::string& name, const std::string& dtype, const std::vector<std::int64_t>& shape,
           const void* data, std::uint64_t nbytes);
  // Finalises every shard (model-XXXXX-of-YYYYY.safetensors) and writes the index.  Idempotent.
  bool close();
  const std::vector<std::string>& shard_files() const { return _files; }

private:
  struct Entry {
    std::string name, dtype;
    std::vector<std::int64_t> shape;
    std::uint64_t offset = 0, nbytes = 0;
  };
  struct Held {                      // a small tensor whose size is not a multiple of 16
    Entry e;
    std::vector<std::uint8_t> bytes;
  };
  struct Shard {
    std::string blob_path;
    int fd = -1;
    std::uint64_t size = 0;
    std::vector<Entry> entries;
    std::vector<Held> held;          // written after everything else, so nothing else is shifted
    std::uint64_t held_bytes = 0;
  };
  static constexpr std::uint64_t kHeldMax = 1ull << 20;
  static constexpr std::uint64_t kHeldTotalMax = 64ull << 20;
  bool current_shard(std::uint64_t incoming);
  bool finish_shard(std::size_t idx, std::size_t total, std::string* file_name);

  std::string _dir;
  std::uint64_t _shard_max;
  std::vector<Shard> _shards;
  std::vector<std::string> _files;
  std::unordered_map<std::string, int> _names;
  bool _closed = false;
};

// Quantizes one bf16 [N,K] weight on the device (the packer of include/vpq.h) and appends its
// three tensors under `prefix` (generative-models/quantize/affine-quantizer.cc:52-84 followed by
// the writer calls of the model quantizer): `.weight` U32 [N,K/8], `.scales`, `.biases` F16 [N,K/64].
bool quantize_and_add(CommandStream& stream, PackWriter& writer, const std::string& prefix,
                      const DeviceBuffer& src_bf16, int K, int N, float clip = 1.0f, std::string* why = nullptr);

}  // namespace vpipe_amd

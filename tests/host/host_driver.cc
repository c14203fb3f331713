// Test driver: plain-C entry points over the C++ host layer (vpipe_amd/host/vpq_host.h), so that
// the Python tests can write quantized-linear call sites in the reference's encoder protocol
// (set_function / set_buffer / set_constant / dispatch / fence) and check them against the oracle.
// Not part of the product; built next to this file.
#include <algorithm>
#include <cstring>
#include <optional>
#include <string>
#include <vector>

#include "vpq_host.h"
#include "vpq_weights.h"

using namespace vpipe_amd;

namespace {

struct Session {
  CommandStream stream;
  ComputeEncoder enc;
  std::vector<ComputeEncoder::ConcurrentScope> scopes;
  std::string reason;
};

}  // namespace

extern "C" {

void* hd_open(void)
{
  Session* s = new Session();
  s->stream = CommandStream::create();
  if (!s->stream.valid()) { delete s; return nullptr; }
  s->enc = s->stream.begin_compute();
  return s;
}

void hd_close(void* h)
{
  Session* s = static_cast<Session*>(h);
  if (s == nullptr) { return; }
  s->scopes.clear();
  s->enc.end();
  delete s;
}

// 1 if `library` holds `function`, 0 otherwise; binds it to the encoder when it does.
int hd_set_function(void* h, const char* library, const char* function)
{
  Session* s = static_cast<Session*>(h);
  QuantLibrary lib = QuantLibrary::load(library);
  QuantFunction fn = lib.function(function);
  s->enc.set_function(fn);
  return fn.valid() ? 1 : 0;
}

void hd_set_buffer(void* h, unsigned index, void* device_ptr, size_t bytes, size_t byte_offset)
{
  Session* s = static_cast<Session*>(h);
  DeviceBuffer b = DeviceBuffer::wrap(device_ptr, bytes);
  s->enc.set_buffer(index, b, byte_offset);
}

void hd_set_constant_i32(void* h, unsigned index, int value)
{
  static_cast<Session*>(h)->enc.set_constant(index, value);
}

void hd_set_constant_f32(void* h, unsigned index, float value)
{
  static_cast<Session*>(h)->enc.set_constant(index, value);
}

void hd_dispatch(void* h, unsigned gx, unsigned gy, unsigned gz, unsigned tx, unsigned ty, unsigned tz)
{
  static_cast<Session*>(h)->enc.dispatch(LaunchDims{gx, gy, gz}, LaunchDims{tx, ty, tz});
}

void hd_scope_begin(void* h)
{
  Session* s = static_cast<Session*>(h);
  s->scopes.push_back(s->enc.concurrent_scope(true));
}

void hd_scope_end(void* h)
{
  Session* s = static_cast<Session*>(h);
  if (!s->scopes.empty()) { s->scopes.pop_back(); }
}

long hd_dispatch_count(void* h) { return static_cast<Session*>(h)->enc.dispatch_count(); }

// 1 = everything committed so far ran; 0 = an error was recorded (text via hd_reason).
int hd_wait_ok(void* h)
{
  Session* s = static_cast<Session*>(h);
  s->reason.clear();
  Fence f = s->stream.commit();
  return f.wait_ok(&s->reason) ? 1 : 0;
}

const char* hd_reason(void* h) { return static_cast<Session*>(h)->reason.c_str(); }

// quant_linear_forward over wrapped device pointers; lora_a may be NULL.
void hd_quant_linear(void* h, void* codes, void* scales, void* qbias, int K, int N, void* x, void* y, int M,
                     void* lora_a, void* lora_b, int rank, float strength, void* lora_t)
{
  Session* s = static_cast<Session*>(h);
  const size_t kb = (size_t)N * K / 2, sb = (size_t)N * (K / 64) * 2;
  DeviceBuffer bc = DeviceBuffer::wrap(codes, kb), bs = DeviceBuffer::wrap(scales, sb), bq = DeviceBuffer::wrap(qbias, sb);
  DeviceBuffer bx = DeviceBuffer::wrap(x, (size_t)M * K * 2), by = DeviceBuffer::wrap(y, (size_t)M * N * 2);
  Linear lin;
  lin.codes = &bc; lin.scales = &bs; lin.qbias = &bq; lin.K = K; lin.N = N;
  if (lora_a != nullptr) {
    DeviceBuffer la = DeviceBuffer::wrap(lora_a, (size_t)rank * K * 2), lb = DeviceBuffer::wrap(lora_b, (size_t)N * rank * 2);
    DeviceBuffer lt = DeviceBuffer::wrap(lora_t, (size_t)M * rank * 2);
    LoraFactors lf;
    lf.a = &la; lf.b = &lb; lf.rank = rank; lf.strength = strength;
    quant_linear_forward(s->stream, lin, bx, 0, by, 0, M, &lf, &lt);
  } else {
    quant_linear_forward(s->stream, lin, bx, 0, by, 0, M);
  }
}

// The same over a pack of another width / group (bits 4 or 8, group 64 or 32), with an adapter.
void hd_quant_linear_fmt(void* h, void* codes, void* scales, void* qbias, int bits, int group, int K, int N, void* x, void* y,
                         int M, void* lora_a, void* lora_b, int rank, float strength, void* lora_t)
{
  Session* s = static_cast<Session*>(h);
  const size_t kb = (size_t)N * K * bits / 8, sb = (size_t)N * (K / group) * 2;
  DeviceBuffer bc = DeviceBuffer::wrap(codes, kb), bs = DeviceBuffer::wrap(scales, sb), bq = DeviceBuffer::wrap(qbias, sb);
  DeviceBuffer bx = DeviceBuffer::wrap(x, (size_t)M * K * 2), by = DeviceBuffer::wrap(y, (size_t)M * N * 2);
  Linear lin;
  lin.codes = &bc; lin.scales = &bs; lin.qbias = &bq; lin.K = K; lin.N = N; lin.bits = bits; lin.group = group;
  DeviceBuffer la = DeviceBuffer::wrap(lora_a, (size_t)rank * K * 2), lb = DeviceBuffer::wrap(lora_b, (size_t)N * rank * 2);
  DeviceBuffer lt = DeviceBuffer::wrap(lora_t, (size_t)M * rank * 2);
  LoraFactors lf;
  lf.a = &la; lf.b = &lb; lf.rank = rank; lf.strength = strength;
  quant_linear_forward(s->stream, lin, bx, 0, by, 0, M, &lf, &lt);
}

// ---- checkpoint container (vpq_weights.h) ---------------------------------------------------

void* hw_open(const char* dir, unsigned long long shard_max_bytes)
{
  return new PackWriter(dir, shard_max_bytes);
}

int hw_add(void* h, const char* name, const char* dtype, const long long* shape, int ndim, const void* data,
           unsigned long long nbytes)
{
  std::vector<std::int64_t> shp(shape, shape + ndim);
  return static_cast<PackWriter*>(h)->add(name, dtype, shp, data, nbytes) ? 1 : 0;
}

// Closes and frees the writer; 1 if every shard and the index were written.
int hw_close(void* h)
{
  PackWriter* w = static_cast<PackWriter*>(h);
  const bool ok = w->close();
  delete w;
  return ok ? 1 : 0;
}

static std::string g_why;
const char* hr_why(void) { return g_why.c_str(); }

void* hr_open(const char* path, int model_dir)
{
  g_why.clear();
  std::optional<PackFile> f = model_dir ? PackFile::open_model(path, &g_why) : PackFile::open(path, &g_why);
  if (!f) { return nullptr; }
  return new PackFile(std::move(*f));
}

void hr_close(void* h) { delete static_cast<PackFile*>(h); }

int hr_count(void* h) { return (int)static_cast<PackFile*>(h)->tensor_names().size(); }

// Name of the i-th tensor (sorted) into buf.
int hr_name(void* h, int i, char* buf, int cap)
{
  std::vector<std::string> names = static_cast<PackFile*>(h)->tensor_names();
  std::sort(names.begin(), names.end());
  if (i < 0 || i >= (int)names.size() || (int)names[i].size() + 1 > cap) { return 0; }
  std::memcpy(buf, names[i].c_str(), names[i].size() + 1);
  return 1;
}

// dtype into dtype_buf (16 bytes), up to 8 dims into shape; out = {ndim, nbytes, offset, shard}.
int hr_info(void* h, const char* name, char* dtype_buf, long long* shape, unsigned long long* out)
{
  const TensorInfo* ti = static_cast<PackFile*>(h)->info(name);
  if (ti == nullptr || ti->shape.size() > 8 || ti->dtype.size() > 15) { return 0; }
  std::memcpy(dtype_buf, ti->dtype.c_str(), ti->dtype.size() + 1);
  for (std::size_t i = 0; i < ti->shape.size(); ++i) { shape[i] = ti->shape[i]; }
  out[0] = ti->shape.size(); out[1] = ti->nbytes; out[2] = ti->offset; out[3] = (unsigned long long)ti->shard;
  return 1;
}

int hr_read(void* h, const char* name, void* dst, unsigned long long cap)
{
  return static_cast<PackFile*>(h)->read_into(name, dst, cap) ? 1 : 0;
}

void hr_alignment(void* h, long long* out4)
{
  const PackFile::Alignment a = static_cast<PackFile*>(h)->alignment();
  out4[0] = (long long)a.tensors; out4[1] = (long long)a.misaligned; out4[2] = a.shards; out4[3] = a.bad_shards;
}

int hr_bits(void* h, const char* prefix, int K) { return static_cast<PackFile*>(h)->affine_bits(prefix, K); }
int hr_group(void* h, const char* prefix, int K) { return static_cast<PackFile*>(h)->affine_group(prefix, K); }

// Quantizes a bf16 [N,K] device tensor and appends `<prefix>.weight/.scales/.biases` to the writer.
int hd_quantize_and_add(void* session, void* writer, const char* prefix, void* src_bf16, int K, int N, float clip)
{
  Session* s = static_cast<Session*>(session);
  DeviceBuffer src = DeviceBuffer::wrap(src_bf16, (size_t)N * K * 2);
  return quantize_and_add(s->stream, *static_cast<PackWriter*>(writer), prefix, src, K, N, clip, &g_why) ? 1 : 0;
}

// Loads one Linear from the reader and runs y[M,N] = x . W^T through quant_linear_forward.
// out_kn receives {K, N}.  The loaded buffers live until the call returns (it waits).
int hd_load_and_run(void* session, void* reader, const char* prefix, int K, void* x, void* y, int M, int* out_kn)
{
  Session* s = static_cast<Session*>(session);
  LoadedLinear lin;
  if (!static_cast<PackFile*>(reader)->load_linear(s->stream, prefix, K, &lin, &g_why)) { return 0; }
  out_kn[0] = lin.K; out_kn[1] = lin.N;
  DeviceBuffer bx = DeviceBuffer::wrap(x, (size_t)M * lin.K * 2), by = DeviceBuffer::wrap(y, (size_t)M * lin.N * 2);
  quant_linear_forward(s->stream, lin.view(), bx, 0, by, 0, M);
  return s->stream.commit().wait_ok(&g_why) ? 1 : 0;
}

}  // extern "C"

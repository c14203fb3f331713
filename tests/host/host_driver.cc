// Test driver: plain-C entry points over the C++ host layer (vpipe_amd/host/vpq_host.h), so that
// the Python tests can write quantized-linear call sites in the reference's encoder protocol
// (set_function / set_buffer / set_constant / dispatch / fence) and check them against the oracle.
// Not part of the product; built next to this file.
#include <cstring>
#include <string>
#include <vector>

#include "vpq_host.h"

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

}  // extern "C"

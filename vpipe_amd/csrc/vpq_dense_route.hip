// The dequant-once route of QMM: the pack is expanded to bf16 [N,K] once (the a1 kernel) and the
// contraction y = x . w_deq^T is a plain dense GEMM, handed to the vendor BLAS.  This is the
// reference's `gemm_mma_` route (generative-models/minimax-h3/metal-minimax-h3-transformer.cc:
// 2020-2160: affine_dequant into a scratch + a dense matrix-unit GEMM); there the expansion costs
// 2*N*K bytes of traffic per call, here the caller may keep the expansion of an immutable weight.
//
// rocBLAS is opened at first use with dlopen, so that the library has no link-time dependency on
// it and every other entry point works without it.  One handle per process, calls serialised by a
// mutex (the handle carries the stream).  Creating the handle allocates: the first call of this
// route is not allocation-free, later ones are.
#include <dlfcn.h>

#include <mutex>
#include <string>

#include "vpq_internal.h"

namespace vpq {

namespace {

// The few rocBLAS declarations this file needs (rocblas/internal/rocblas-types.h, -functions.h).
typedef void* rb_handle;
constexpr int kOpNone = 111, kOpTranspose = 112;
constexpr int kBf16 = 168, kF16 = 150, kF32 = 151;
typedef int (*rb_create_handle_t)(rb_handle*);
typedef int (*rb_set_stream_t)(rb_handle, hipStream_t);
typedef int (*rb_gemm_ex_t)(rb_handle, int, int, int, int, int, const void*, const void*, int, int, const void*, int,
                            int, const void*, const void*, int, int, void*, int, int, int, int, int32_t, uint32_t);

struct Rocblas {
  std::mutex mu;
  bool tried = false;
  void* lib = nullptr;
  rb_handle handle = nullptr;
  rb_set_stream_t set_stream = nullptr;
  rb_gemm_ex_t gemm_ex = nullptr;
  std::string error;
};

Rocblas& rocblas()
{
  static Rocblas r;
  return r;
}

bool open_locked(Rocblas& r)
{
  if (r.tried) { return r.handle != nullptr; }
  r.tried = true;
  const char* names[] = {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"};
  for (const char* n : names) {
    r.lib = dlopen(n, RTLD_NOW | RTLD_GLOBAL);
    if (r.lib != nullptr) { break; }
  }
  if (r.lib == nullptr) {
    r.error = std::string("rocBLAS not found: ") + dlerror();
    return false;
  }
  rb_create_handle_t create = reinterpret_cast<rb_create_handle_t>(dlsym(r.lib, "rocblas_create_handle"));
  r.set_stream = reinterpret_cast<rb_set_stream_t>(dlsym(r.lib, "rocblas_set_stream"));
  r.gemm_ex = reinterpret_cast<rb_gemm_ex_t>(dlsym(r.lib, "rocblas_gemm_ex"));
  if (create == nullptr || r.set_stream == nullptr || r.gemm_ex == nullptr) {
    r.error = "rocBLAS lacks rocblas_create_handle / rocblas_set_stream / rocblas_gemm_ex";
    return false;
  }
  rb_handle h = nullptr;
  const int st = create(&h);
  if (st != 0 || h == nullptr) {
    r.error = "rocblas_create_handle failed with status " + std::to_string(st);
    return false;
  }
  r.handle = h;
  return true;
}

}  // namespace

// y[M,N] = x[M,K] . b[N,K]^T, bf16 operands, fp32 accumulation, bf16 result.  Returns 0, or a
// negative value with *why set: -1 rocBLAS unavailable, -2 the GEMM call failed.
int dense_gemm_bf16(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K,
                    std::string* why)
{
  return dense_gemm_elt(st, x, b, y, M, N, K, false, why);
}

// The same with IEEE binary16 operands and result when f16 is set.
int dense_gemm_elt(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K, bool f16,
                   std::string* why)
{
  const int dt = f16 ? kF16 : kBf16;
  Rocblas& r = rocblas();
  std::lock_guard<std::mutex> lock(r.mu);
  if (!open_locked(r)) {
    if (why) { *why = r.error; }
    return -1;
  }
  int rc = r.set_stream(r.handle, st);
  if (rc == 0) {
    // Column-major view: y^T (N x M, ld N) = b (as K x N, ld K)^T . x (as K x M, ld K).
    const float alpha = 1.0f, beta = 0.0f;
    rc = r.gemm_ex(r.handle, kOpTranspose, kOpNone, N, M, K, &alpha, b, dt, K, x, dt, K, &beta, y, dt, N, y, dt, N, kF32, 0,
                   0, 0u);
  }
  if (rc != 0) {
    if (why) { *why = "rocBLAS status " + std::to_string(rc); }
    return -2;
  }
  return 0;
}

}  // namespace vpq

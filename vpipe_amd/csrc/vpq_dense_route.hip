// The dequant-once route of QMM: the pack is expanded to a dense [N,K] matrix once (the a1 kernel) and the
// contraction y = x . w_deq^T is a plain dense GEMM on the library's own large-tile kernel.  This is the
// reference's `gemm_mma_` route (generative-models/minimax-h3/metal-minimax-h3-transformer.cc:2020-2160:
// affine_dequant into a scratch + the dense matrix-unit GEMM of gpu-kernels/metal/gemm/dense_gemm_mma.metal);
// there the expansion costs 2*N*K bytes of traffic per call, here the caller may keep the expansion of an
// immutable weight.  Nothing here allocates, synchronises or opens another library.
#include <string>

#include "vpq_internal.h"

namespace vpq {

// y[M,N] = x[M,K] . b[N,K]^T, bf16 operands, fp32 accumulation, bf16 result.  Returns 0, or -2 with *why set
// when the launch failed or the shape is outside what the kernel takes.
int dense_gemm_bf16(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K, int cu_count,
                    std::string* why)
{
  return dense_gemm_elt(st, x, b, y, M, N, K, false, cu_count, why);
}

// The same with IEEE binary16 operands and result when f16 is set.
int dense_gemm_elt(hipStream_t st, const uint16_t* x, const uint16_t* b, uint16_t* y, int M, int N, int K, bool f16,
                   int cu_count, std::string* why)
{
  if (!dense_gemm_supports(M, N, K)) {
    if (why) { *why = "dense GEMM: K must be a multiple of 32 and the matrices below 4 GB"; }
    return -2;
  }
  const hipError_t e = launch_dense_gemm(st, x, b, y, M, N, K, f16, cu_count);
  if (e != hipSuccess) {
    if (why) { *why = hipGetErrorString(e); }
    return -2;
  }
  return 0;
}

}  // namespace vpq

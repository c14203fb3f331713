// Implementation of the C++ host layer over the C ABI (see vpq_host.h).
#include "vpq_host.h"

#include <hip/hip_runtime_api.h>

#include <cstring>
#include <utility>

#include "vpq.h"

namespace vpipe_amd {

// ---------------------------------------------------------------- DeviceBuffer
DeviceBuffer::DeviceBuffer(DeviceBuffer&& o) noexcept : _ptr(o._ptr), _bytes(o._bytes), _owned(o._owned)
{
  o._ptr = nullptr; o._bytes = 0; o._owned = false;
}

DeviceBuffer& DeviceBuffer::operator=(DeviceBuffer&& o) noexcept
{
  if (this != &o) {
    if (_owned && _ptr) { (void)hipFree(_ptr); }
    _ptr = o._ptr; _bytes = o._bytes; _owned = o._owned;
    o._ptr = nullptr; o._bytes = 0; o._owned = false;
  }
  return *this;
}

DeviceBuffer::~DeviceBuffer()
{
  if (_owned && _ptr) { (void)hipFree(_ptr); }
}

DeviceBuffer DeviceBuffer::allocate(std::size_t bytes)
{
  DeviceBuffer b;
  void* p = nullptr;
  if (bytes > 0 && hipMalloc(&p, bytes) == hipSuccess) {
    b._ptr = p; b._bytes = bytes; b._owned = true;
  } else {
    (void)hipGetLastError();
  }
  return b;
}

DeviceBuffer DeviceBuffer::wrap(void* device_ptr, std::size_t bytes) noexcept
{
  DeviceBuffer b;
  b._ptr = device_ptr; b._bytes = device_ptr ? bytes : 0; b._owned = false;
  return b;
}

bool DeviceBuffer::upload(const void* host, std::size_t bytes, std::size_t byte_offset) const
{
  if (empty() || byte_offset + bytes > _bytes) { return false; }
  return hipMemcpy(static_cast<char*>(_ptr) + byte_offset, host, bytes, hipMemcpyHostToDevice) == hipSuccess;
}

bool DeviceBuffer::download(void* host, std::size_t bytes, std::size_t byte_offset) const
{
  if (empty() || byte_offset + bytes > _bytes) { return false; }
  return hipMemcpy(host, static_cast<const char*>(_ptr) + byte_offset, bytes, hipMemcpyDeviceToHost) == hipSuccess;
}

// ---------------------------------------------------------------- QuantLibrary
namespace {

struct FnEntry {
  const char* library;
  const char* function;
  QuantKernel kind;
  QuantFormat format = QuantFormat::W4G64;
};

// Function names of the reference's bf16 metallibs that this path serves.
const FnEntry kFunctions[] = {
    {"affine_dequant_bf16", "affine_dequant_w4g64", QuantKernel::Dequant},
    {"affine_qmv_bf16", "affine_qmv_w4g64", QuantKernel::Qmv},
    {"affine_qmv_bf16", "affine_qmv_w4g64_add", QuantKernel::QmvAdd},
    {"affine_qmv_bf16", "affine_qmv_batch_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch4_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch4_xp_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch8_xp_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch8_xp2_w4g64", QuantKernel::QmvBatch},
    // the other tilings of the same batched GEMV (gpu-kernels/metal/quant/affine_qmv.metal:1911-2549: threadgroup-
    // staged x, hoisted nibbles, weight packs in registers; `xh16` multiplies in half there and in fp32 here)
    {"affine_qmv_bf16", "affine_qmv_batch8_xp1_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch8_tg_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch8_tg4_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch8_xd_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch8_xh_w4g64", QuantKernel::QmvBatch},
    {"affine_qmv_bf16", "affine_qmv_batch8_xh16_w4g64", QuantKernel::QmvBatch},
    // batched gated GEMVs (:2336-2354, 2854-2872, 3003): slot 7 = m_total
    {"affine_qmv_bf16", "affine_qmv_batch_swiglu_w4g64", QuantKernel::QmvBatchSwiglu},
    {"affine_qmv_bf16", "affine_qmv_batch4_swiglu_w4g64", QuantKernel::QmvBatchSwiglu},
    {"affine_qmv_bf16", "affine_qmv_batch4_xp_swiglu_w4g64", QuantKernel::QmvBatchSwiglu},
    {"affine_qmv_bf16", "affine_qmv_batch8_xp2_swiglu_w4g64", QuantKernel::QmvBatchSwiglu},
    {"affine_qmv_bf16", "affine_qmv_batch_geglu_w4g64", QuantKernel::QmvBatchGeglu},
    // batched GEMVs of the twins (:1718-1736, 2328-2334, 2725-2745, 3026)
    {"affine_qmv_bf16", "affine_qmv_batch_w8g64", QuantKernel::QmvBatch, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_batch4_w8g64", QuantKernel::QmvBatch, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_batch4_xp_w8g64", QuantKernel::QmvBatch, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_batch8_xp2_w8g64", QuantKernel::QmvBatch, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_batch8_tg4_w8g64", QuantKernel::QmvBatch, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_batch8_xd_w8g64", QuantKernel::QmvBatch, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_batch_w4g32", QuantKernel::QmvBatch, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_qmv_batch_geglu_w4g32", QuantKernel::QmvBatchGeglu, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_qmv_qkv_w4g64", QuantKernel::QmvQkv},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w4g64", QuantKernel::Qmm},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w4g64_bm64", QuantKernel::Qmm},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w4g64_bm128", QuantKernel::Qmm},
    {"affine_qmm_mma_bf16", "affine_qmm_mma_w4g64", QuantKernel::Qmm},
    {"affine_qmv_bf16", "affine_qmv_swiglu_w4g64", QuantKernel::QmvSwiglu},
    {"affine_qmv_bf16", "affine_qmv_geglu_w4g64", QuantKernel::QmvGeglu},
    {"affine_qmv_bf16", "affine_qmv_gelu_mul_w4g64", QuantKernel::QmvGeluMul},
    {"affine_qmm_steel_bf16", "affine_qmm_geglu_w4g64", QuantKernel::QmmGeglu},
    {"llm_elementwise_bf16", "dequant_embed_gather_f16", QuantKernel::EmbedGather},
    {"llm_elementwise_bf16", "argmax_f16", QuantKernel::Argmax},
    {"llm_elementwise_bf16", "argmax_partial_f16", QuantKernel::ArgmaxPartial},
    {"llm_elementwise_bf16", "argmax_combine_f16", QuantKernel::ArgmaxCombine},
    {"llm_elementwise_bf16", "sample_topp_f16", QuantKernel::SampleTopp},
    {"affine_qmv_bf16", "affine_gather_qmv_swiglu_w4g64", QuantKernel::GatherSwiglu},
    {"affine_qmv_bf16", "affine_gather_qmv_geglu_w4g64", QuantKernel::GatherGeglu},
    {"affine_qmv_bf16", "affine_gather_down_qmv_w4g64", QuantKernel::GatherDown},
    {"affine_qmm_steel_bf16", "affine_qmm_grouped_swiglu_w4g64", QuantKernel::GroupedSwiglu},
    {"affine_qmm_steel_bf16", "affine_qmm_grouped_geglu_w4g64", QuantKernel::GroupedGeglu},
    {"affine_qmm_steel_bf16", "affine_qmm_grouped_w4g64", QuantKernel::GroupedDown},
    {"affine_qmv_bf16", "affine_grouped_swiglu_w4g64", QuantKernel::SortedSwiglu},
    {"affine_qmv_bf16", "affine_grouped_down_w4g64", QuantKernel::SortedDown},
    {"affine_qmv_bf16", "affine_gather_qmv_swiglu_w4w8g64", QuantKernel::GatherSplit48},
    {"affine_qmv_bf16", "affine_gather_qmv_swiglu_w8w4g64", QuantKernel::GatherSplit84},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64", QuantKernel::QmmSwiglu},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_bm64", QuantKernel::QmmSwiglu},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_bm128", QuantKernel::QmmSwiglu},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_bm64_rs", QuantKernel::QmmSwiglu},
    // 8-bit and group-32 twins (gpu-kernels/metal/quant/affine_dequant.metal:68-97, 196-228;
    // affine_qmv.metal:305-403, 1451-1490, 3034-3050, 3122-3140; affine_qmm_steel.metal:1601-)
    {"affine_dequant_bf16", "affine_dequant_w8g64", QuantKernel::Dequant, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_w8g64", QuantKernel::Qmv, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_w8g64_add", QuantKernel::QmvAdd, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_moe_gate_w8g64", QuantKernel::MoeGate, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_gelu_mul_w8g64", QuantKernel::QmvGeluMul, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_gelu_mul_w4g32", QuantKernel::QmvGeluMul, QuantFormat::W4G32},
    {"affine_dequant_bf16", "affine_requant_w8_to_w4_g64", QuantKernel::Requant84, QuantFormat::W8G64},
    // the packer at every width and group (gpu-kernels/metal/quant/affine_dequant.metal:243-301); the reference's
    // quantizer loads it from the binary16 library (generative-models/quantize/affine-quantizer.cc:25)
    {"affine_dequant_bf16", "affine_quant_w4_g64", QuantKernel::QuantizeBf16, QuantFormat::W4G64},
    {"affine_dequant_bf16", "affine_quant_w4_g32", QuantKernel::QuantizeBf16, QuantFormat::W4G32},
    {"affine_dequant_bf16", "affine_quant_w8_g64", QuantKernel::QuantizeBf16, QuantFormat::W8G64},
    {"affine_dequant_bf16", "affine_quant_w8_g32", QuantKernel::QuantizeBf16, QuantFormat::W8G32},
    {"affine_dequant", "affine_quant_w4_g64", QuantKernel::QuantizeF16, QuantFormat::W4G64},
    {"affine_dequant", "affine_quant_w4_g32", QuantKernel::QuantizeF16, QuantFormat::W4G32},
    {"affine_dequant", "affine_quant_w8_g64", QuantKernel::QuantizeF16, QuantFormat::W8G64},
    {"affine_dequant", "affine_quant_w8_g32", QuantKernel::QuantizeF16, QuantFormat::W8G32},
    // Tiling variants the reference keeps beside its defaults (affine_qmv.metal:3072-3118: rows per simdgroup / packs
    // per thread of the same GEMV) and its plain QMM (affine_qmm.metal:64-174): the same mathematics, served by the
    // same kernels (the plain QMM exists in the binary16 build only).  The `_acc16` GEMMs accumulate in fp32 in the
    // bf16 library (affine_qmm_steel.metal:50-56), so there they are the base functions under another name; the
    // binary16 library's half accumulation is not served.
    {"affine_qmv_bf16", "affine_qmv_w4g64_r8p2", QuantKernel::Qmv},
    {"affine_qmv_bf16", "affine_qmv_w8g64_r8p2", QuantKernel::Qmv, QuantFormat::W8G64},
    {"affine_qmm", "affine_qmm_w4g64", QuantKernel::Qmm, QuantFormat::W4G64F16},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w4g64_bm64_acc16", QuantKernel::Qmm},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_acc16", QuantKernel::QmmSwiglu},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_bm64_acc16", QuantKernel::QmmSwiglu},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w4g64_bm64_rs_acc16", QuantKernel::QmmSwiglu},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w8g64_bm64_acc16", QuantKernel::Qmm, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_acc16", QuantKernel::QmmSwiglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_bm64_acc16", QuantKernel::QmmSwiglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_bm64_rs_acc16", QuantKernel::QmmSwiglu, QuantFormat::W8G64},
    {"affine_dequant_bf16", "affine_dequant_w8g32", QuantKernel::Dequant, QuantFormat::W8G32},
    {"affine_qmv_bf16", "affine_qmv_w8g32", QuantKernel::Qmv, QuantFormat::W8G32},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w8g32", QuantKernel::Qmm, QuantFormat::W8G32},
    {"affine_qmv_bf16", "affine_qmv_qkv_w8g64", QuantKernel::QmvQkv, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_qkv_rms_w4g64", QuantKernel::QmvQkvRms},
    {"affine_qmv_bf16", "affine_qmv_qkv_rms_w4g32", QuantKernel::QmvQkvRms, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_qmv_qkv_rms_w8g64", QuantKernel::QmvQkvRms, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_qkv_w4g32", QuantKernel::QmvQkv, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_grouped_swiglu_w8g64", QuantKernel::SortedSwiglu, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_grouped_down_w8g64", QuantKernel::SortedDown, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w8g64", QuantKernel::Qmm, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w8g64_bm64", QuantKernel::Qmm, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w8g64_bm128", QuantKernel::Qmm, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64", QuantKernel::QmmSwiglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_bm64", QuantKernel::QmmSwiglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_bm128", QuantKernel::QmmSwiglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_swiglu_w8g64_bm64_rs", QuantKernel::QmmSwiglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_geglu_w8g64", QuantKernel::QmmGeglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_grouped_swiglu_w8g64", QuantKernel::GroupedSwiglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_grouped_geglu_w8g64", QuantKernel::GroupedGeglu, QuantFormat::W8G64},
    {"affine_qmm_steel_bf16", "affine_qmm_grouped_w8g64", QuantKernel::GroupedDown, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_swiglu_w8g64", QuantKernel::QmvSwiglu, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_qmv_geglu_w8g64", QuantKernel::QmvGeglu, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_gather_qmv_swiglu_w8g64", QuantKernel::GatherSwiglu, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_gather_qmv_geglu_w8g64", QuantKernel::GatherGeglu, QuantFormat::W8G64},
    {"affine_qmv_bf16", "affine_gather_down_qmv_w8g64", QuantKernel::GatherDown, QuantFormat::W8G64},
    // IEEE binary16 build (VPIPE_ELT = half; generative-models/qwen3/metal-qwen-model.cc:771-772: the library
    // names without the suffix)
    {"affine_dequant", "affine_dequant_w4g64", QuantKernel::Dequant, QuantFormat::W4G64F16},
    // the 8-bit functions of the binary16 build (the codec's: generative-models/moss/metal-moss-codec.cc:181-183, 579-581)
    {"affine_dequant", "affine_dequant_w8g64", QuantKernel::Dequant, QuantFormat::W8G64F16},
    {"affine_dequant", "affine_dequant_w8g32", QuantKernel::Dequant, QuantFormat::W8G32F16},
    {"affine_qmm_steel", "affine_qmm_steel_w8g64", QuantKernel::Qmm, QuantFormat::W8G64F16},
    {"affine_qmm_steel", "affine_qmm_steel_w8g32", QuantKernel::Qmm, QuantFormat::W8G32F16},
    {"affine_qmv", "affine_qmv_w4g64", QuantKernel::Qmv, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_w4g64_add", QuantKernel::QmvAdd, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_swiglu_w4g64", QuantKernel::QmvSwiglu, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_geglu_w4g64", QuantKernel::QmvGeglu, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_qkv_w4g64", QuantKernel::QmvQkv, QuantFormat::W4G64F16},
    // the batched GEMVs of the binary16 build (rows = m_total in slot 7)
    {"affine_qmv", "affine_qmv_batch_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch4_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch4_xp_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_xp_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_xp2_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_xp1_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_tg_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_tg4_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_xd_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_xh_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_xh16_w4g64", QuantKernel::QmvBatch, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch_swiglu_w4g64", QuantKernel::QmvBatchSwiglu, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch4_swiglu_w4g64", QuantKernel::QmvBatchSwiglu, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch4_xp_swiglu_w4g64", QuantKernel::QmvBatchSwiglu, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch8_xp2_swiglu_w4g64", QuantKernel::QmvBatchSwiglu, QuantFormat::W4G64F16},
    {"affine_qmv", "affine_qmv_batch_geglu_w4g64", QuantKernel::QmvBatchGeglu, QuantFormat::W4G64F16},
    {"affine_qmm_steel", "affine_qmm_steel_w4g64", QuantKernel::Qmm, QuantFormat::W4G64F16},
    {"affine_qmm_steel", "affine_qmm_steel_w4g64_bm64", QuantKernel::Qmm, QuantFormat::W4G64F16},
    {"affine_qmm_steel", "affine_qmm_steel_w4g64_bm128", QuantKernel::Qmm, QuantFormat::W4G64F16},
    {"affine_qmm_steel", "affine_qmm_swiglu_w4g64", QuantKernel::QmmSwiglu, QuantFormat::W4G64F16},
    {"affine_qmm_steel", "affine_qmm_geglu_w4g64", QuantKernel::QmmGeglu, QuantFormat::W4G64F16},
    {"affine_dequant_bf16", "affine_dequant_w4g32", QuantKernel::Dequant, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_qmv_w4g32", QuantKernel::Qmv, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_qmv_w4g32_add", QuantKernel::QmvAdd, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_qmv_w4g32_q40", QuantKernel::Qmv, QuantFormat::W4G32Q40},
    {"affine_qmv_bf16", "affine_qmv_w4g32_add_q40", QuantKernel::QmvAdd, QuantFormat::W4G32Q40},
    {"affine_qmm_steel_bf16", "affine_qmm_steel_w4g32", QuantKernel::Qmm, QuantFormat::W4G32},
    {"affine_qmm_steel_bf16", "affine_qmm_geglu_w4g32", QuantKernel::QmmGeglu, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_qmv_geglu_w4g32", QuantKernel::QmvGeglu, QuantFormat::W4G32},
    {"affine_qmv_bf16", "affine_qmv_geglu_w4g32_q40", QuantKernel::QmvGeglu, QuantFormat::W4G32Q40},
};

}  // namespace

QuantLibrary QuantLibrary::load(const std::string& name)
{
  QuantLibrary lib;
  for (const FnEntry& e : kFunctions) {
    if (name == e.library) { lib._name = name; break; }
  }
  return lib;
}

QuantFunction QuantLibrary::function(const std::string& fn_name) const
{
  QuantFunction fn;
  for (const FnEntry& e : kFunctions) {
    if (_name == e.library && fn_name == e.function) {
      fn._kind = e.kind;
      fn._format = e.format;
      fn._name = fn_name;
      break;
    }
  }
  return fn;
}

// ---------------------------------------------------------------- CommandStream
CommandStream::CommandStream(CommandStream&& o) noexcept { *this = std::move(o); }

CommandStream& CommandStream::operator=(CommandStream&& o) noexcept
{
  if (this != &o) {
    release();
    _main = o._main; _owns_main = o._owns_main; _valid = o._valid;
    _fork_event = o._fork_event;
    for (int i = 0; i < kSideStreams; ++i) { _side[i] = o._side[i]; _join_event[i] = o._join_event[i]; }
    _ws = std::move(o._ws);
    _error = std::move(o._error);
    o._main = nullptr; o._owns_main = false; o._valid = false; o._fork_event = nullptr;
    for (int i = 0; i < kSideStreams; ++i) { o._side[i] = nullptr; o._join_event[i] = nullptr; }
  }
  return *this;
}

CommandStream::~CommandStream() { release(); }

void CommandStream::release()
{
  if (!_valid) { return; }
  (void)hipStreamSynchronize(static_cast<hipStream_t>(_main));
  for (int i = 0; i < kSideStreams; ++i) {
    if (_side[i]) { (void)hipStreamDestroy(static_cast<hipStream_t>(_side[i])); _side[i] = nullptr; }
    if (_join_event[i]) { (void)hipEventDestroy(static_cast<hipEvent_t>(_join_event[i])); _join_event[i] = nullptr; }
  }
  if (_fork_event) { (void)hipEventDestroy(static_cast<hipEvent_t>(_fork_event)); _fork_event = nullptr; }
  if (_owns_main && _main) { (void)hipStreamDestroy(static_cast<hipStream_t>(_main)); }
  _main = nullptr;
  _valid = false;
}

CommandStream CommandStream::create()
{
  CommandStream s;
  if (vpq_init() != VPQ_OK) { return s; }
  hipStream_t st = nullptr;
  if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) {
    (void)hipGetLastError();
    return s;
  }
  s._main = st; s._owns_main = true; s._valid = true;
  return s;
}

CommandStream CommandStream::adopt(void* hip_stream)
{
  CommandStream s;
  if (vpq_init() != VPQ_OK) { return s; }
  s._main = hip_stream; s._owns_main = false; s._valid = true;
  return s;
}

bool CommandStream::ensure_side_streams()
{
  if (_fork_event) { return true; }
  hipEvent_t ev = nullptr;
  if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) { return false; }
  _fork_event = ev;
  for (int i = 0; i < kSideStreams; ++i) {
    hipStream_t st = nullptr;
    hipEvent_t je = nullptr;
    if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&je, hipEventDisableTiming) != hipSuccess) {
      return false;
    }
    _side[i] = st;
    _join_event[i] = je;
  }
  return true;
}

void* CommandStream::qmv_workspace(std::size_t bytes)
{
  if (bytes == 0) { return nullptr; }
  if (_ws.size() < bytes) {
    // Work already queued may still use the old scratch: drain before replacing it.
    (void)hipStreamSynchronize(static_cast<hipStream_t>(_main));
    _ws = DeviceBuffer::allocate(bytes);
    if (_ws.empty()) { return nullptr; }
    if (hipMemset(_ws.data(), 0, bytes) != hipSuccess) { _ws = DeviceBuffer(); return nullptr; }
  }
  return _ws.data();
}

void CommandStream::record_error(int status, const std::string& what)
{
  if (_error.empty()) {
    _error = what + ": " + vpq_status_string(status);
    if (status == VPQ_ERR_DEVICE) { _error += std::string(" (") + vpq_last_device_error() + ")"; }
  }
}

Fence CommandStream::commit()
{
  Fence f;
  f._stream = _valid ? this : nullptr;
  return f;
}

bool Fence::wait_ok(std::string* reason)
{
  if (_stream == nullptr) {
    if (reason) { *reason = "empty fence"; }
    return false;
  }
  const hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(_stream->_main));
  if (e != hipSuccess && _stream->_error.empty()) { _stream->_error = std::string("device: ") + hipGetErrorString(e); }
  if (!_stream->_error.empty()) {
    if (reason) { *reason = _stream->_error; }
    _stream->_error.clear();
    return false;
  }
  return true;
}

// ---------------------------------------------------------------- ComputeEncoder
ComputeEncoder::ComputeEncoder(ComputeEncoder&& o) noexcept { *this = std::move(o); }

ComputeEncoder& ComputeEncoder::operator=(ComputeEncoder&& o) noexcept
{
  if (this != &o) {
    end();
    _stream = o._stream; _fn = o._fn; _n_dispatch = o._n_dispatch;
    _scope_depth = o._scope_depth; _scope_next = o._scope_next; _scope_used = o._scope_used;
    for (unsigned i = 0; i < kSlots; ++i) { _slots[i] = o._slots[i]; }
    o._stream = nullptr;
  }
  return *this;
}

ComputeEncoder::~ComputeEncoder() { end(); }

void ComputeEncoder::end() { _stream = nullptr; }

void ComputeEncoder::set_function(const QuantFunction& fn)
{
  if (!valid()) { return; }
  _fn = fn;
  for (unsigned i = 0; i < kSlots; ++i) { _slots[i] = Slot(); }
}

void ComputeEncoder::set_buffer(unsigned index, const DeviceBuffer& buf, std::size_t byte_offset)
{
  if (!valid() || index >= kSlots || buf.empty()) { return; }
  if (byte_offset > buf.size()) {
    _stream->record_error(VPQ_ERR_BAD_SHAPE, "set_buffer offset beyond the buffer");
    return;
  }
  _slots[index].ptr = static_cast<char*>(buf.data()) + byte_offset;
  _slots[index].bytes = buf.size() - byte_offset;
  _slots[index].is_buffer = true;
  _slots[index].is_const = false;
}

void ComputeEncoder::set_constant_bytes(unsigned index, const void* bytes, std::size_t size)
{
  if (!valid() || index >= kSlots || bytes == nullptr) { return; }
  Slot& s = _slots[index];
  s = Slot();
  s.is_const = true;
  if (size == 4) {
    std::int32_t v; std::memcpy(&v, bytes, 4); s.ivalue = v;
    std::memcpy(&s.fvalue, bytes, 4);
  } else if (size == 8) {
    std::int64_t v; std::memcpy(&v, bytes, 8); s.ivalue = v;
  } else {
    s.is_const = false;   // the kernels of this path take only int / float scalars
  }
}

ComputeEncoder::ConcurrentScope::ConcurrentScope(ComputeEncoder* e, bool active) noexcept
{
  if (e == nullptr || !e->valid() || !active) { return; }
  if (e->_scope_depth == 0) {
    CommandStream* s = e->_stream;
    if (!s->ensure_side_streams()) {
      (void)hipGetLastError();
      return;   // stays serial
    }
    (void)hipEventRecord(static_cast<hipEvent_t>(s->_fork_event), static_cast<hipStream_t>(s->_main));
    e->_scope_next = 0;
    e->_scope_used = 0;
  }
  ++e->_scope_depth;
  _e = e;
}

ComputeEncoder::ConcurrentScope::~ConcurrentScope()
{
  if (_e == nullptr || !_e->valid()) { return; }
  if (--_e->_scope_depth == 0) {
    CommandStream* s = _e->_stream;
    for (int i = 0; i < _e->_scope_used; ++i) {
      (void)hipEventRecord(static_cast<hipEvent_t>(s->_join_event[i]), static_cast<hipStream_t>(s->_side[i]));
      (void)hipStreamWaitEvent(static_cast<hipStream_t>(s->_main), static_cast<hipEvent_t>(s->_join_event[i]), 0);
    }
    _e->_scope_used = 0;
  }
}

void ComputeEncoder::dispatch(LaunchDims grid, LaunchDims /*threads_per_threadgroup*/)
{
  if (!valid()) { return; }
  CommandStream* s = _stream;
  if (!_fn.valid()) {
    s->record_error(VPQ_ERR_NULL_POINTER, "dispatch without a function");
    return;
  }
  auto buf = [&](unsigned i) -> void* { return _slots[i].is_buffer ? _slots[i].ptr : nullptr; };
  auto has_int = [&](unsigned i) { return _slots[i].is_const; };
  auto ival = [&](unsigned i) { return static_cast<int>(_slots[i].ivalue); };

  // Inside a concurrent scope the first dispatch stays on the main stream, the following ones
  // go to side streams that start after everything queued before the scope.
  hipStream_t st = static_cast<hipStream_t>(s->_main);
  const bool in_scope = _scope_depth > 0;
  if (in_scope && _scope_next > 0) {
    const int side = (_scope_next - 1) % CommandStream::kSideStreams;
    st = static_cast<hipStream_t>(s->_side[side]);
    if (side >= _scope_used) {
      (void)hipStreamWaitEvent(st, static_cast<hipEvent_t>(s->_fork_event), 0);
      _scope_used = side + 1;
    }
  }
  if (in_scope) { ++_scope_next; }

  int status = VPQ_OK;
  const QuantKernel kind = _fn.kind();
  const QuantFormat fmt = _fn.format();
  if (kind == QuantKernel::QuantizeBf16 || kind == QuantKernel::QuantizeF16) {
    // gpu-kernels/metal/quant/affine_dequant.metal:287-301: 0:x 1:w 2:scales 3:biases 4:K 5:N 6:clip
    const int bits = (fmt == QuantFormat::W8G64 || fmt == QuantFormat::W8G32) ? 8 : 4;
    const int group = (fmt == QuantFormat::W4G32 || fmt == QuantFormat::W8G32) ? 32 : 64;
    status = (!buf(0) || !buf(1) || !buf(2) || !buf(3) || !has_int(4) || !has_int(5))
                 ? VPQ_ERR_NULL_POINTER
                 : vpq_quantize(st, bits, group, kind == QuantKernel::QuantizeF16 ? 1 : 0, static_cast<const uint16_t*>(buf(0)),
                                static_cast<uint32_t*>(buf(1)), static_cast<uint16_t*>(buf(2)), static_cast<uint16_t*>(buf(3)),
                                ival(4), ival(5), _slots[6].is_const ? _slots[6].fvalue : 1.0f);
  } else if (fmt != QuantFormat::W4G64 && kind != QuantKernel::QmvQkv && kind != QuantKernel::QmvQkvRms) {
    // The 8-bit and group-32 twins keep the slot layout of the 4-bit group-64 functions:
    // dequant 0:w 1:scales 2:biases 3:w_deq 4:K 5:N; QMV 0:w 1:scales 2:biases 3:x 4:y 5:K 6:N [7:residual],
    // rows from grid.x.  The Q4_0 forms ignore slot 2.
    const bool q40 = fmt == QuantFormat::W4G32Q40;
    const uint32_t* w = static_cast<const uint32_t*>(buf(0));
    const uint16_t* sc = static_cast<const uint16_t*>(buf(1));
    const uint16_t* bi = static_cast<const uint16_t*>(buf(2));
    if (kind == QuantKernel::MoeGate) {
      // gpu-kernels/metal/quant/affine_qmv.metal:1327-1349: grid {32, M, 1}
      status = (!w || !sc || !bi || !buf(3) || !buf(4) || !has_int(5))
                   ? VPQ_ERR_NULL_POINTER
                   : vpq_moe_gate_w8g64_bf16(st, w, sc, bi, static_cast<const uint16_t*>(buf(3)),
                                             static_cast<uint16_t*>(buf(4)), ival(5), static_cast<int>(grid.y));
    } else if (kind == QuantKernel::Requant84) {
      // gpu-kernels/metal/quant/affine_dequant.metal:134-186: 0:w8 1:s8 2:b8 3:w4 4:s4 5:b4 6:K 7:N
      status = (!w || !sc || !bi || !buf(3) || !buf(4) || !buf(5) || !has_int(6) || !has_int(7))
                   ? VPQ_ERR_NULL_POINTER
                   : vpq_requant_w8_to_w4_g64_bf16(st, w, sc, bi, static_cast<uint32_t*>(buf(3)),
                                                   static_cast<uint16_t*>(buf(4)), static_cast<uint16_t*>(buf(5)), ival(6),
                                                   ival(7));
    } else if (kind == QuantKernel::QmvGeluMul) {
      // gpu-kernels/metal/quant/affine_qmv.metal:769-805: the slots of the group-64 4-bit form, 7 = the multiplier
      if (!w || !sc || !bi || !buf(3) || !buf(4) || !has_int(5) || !has_int(6) || !buf(7)) {
        status = VPQ_ERR_NULL_POINTER;
      } else if (fmt == QuantFormat::W8G64) {
        status = vpq_qmv_gelu_mul_w8g64_bf16(st, w, sc, bi, static_cast<const uint16_t*>(buf(3)),
                                             static_cast<uint16_t*>(buf(4)), ival(5), ival(6),
                                             static_cast<const uint16_t*>(buf(7)));
      } else {
        status = vpq_qmv_gelu_mul_w4g32_bf16(st, w, sc, bi, static_cast<const uint16_t*>(buf(3)),
                                             static_cast<uint16_t*>(buf(4)), ival(5), ival(6),
                                             static_cast<const uint16_t*>(buf(7)), 0);
      }
    } else if (kind == QuantKernel::Dequant) {
      if (!w || !sc || !bi || !buf(3) || !has_int(4) || !has_int(5)) {
        status = VPQ_ERR_NULL_POINTER;
      } else if (fmt == QuantFormat::W4G64F16) {
        status = vpq_dequant_w4g64_f16(st, w, sc, bi, static_cast<uint16_t*>(buf(3)), ival(4), ival(5));
      } else if (fmt == QuantFormat::W8G64F16 || fmt == QuantFormat::W8G32F16) {
        status = vpq_dequant_w8_f16(st, fmt == QuantFormat::W8G64F16 ? 64 : 32, w, sc, bi, static_cast<uint16_t*>(buf(3)),
                                    ival(4), ival(5));
      } else if (fmt == QuantFormat::W8G64) {
        status = vpq_dequant_w8g64_bf16(st, w, sc, bi, static_cast<uint16_t*>(buf(3)), ival(4), ival(5));
      } else if (fmt == QuantFormat::W8G32) {
        status = vpq_dequant_w8g32_bf16(st, w, sc, bi, static_cast<uint16_t*>(buf(3)), ival(4), ival(5));
      } else {
        status = vpq_dequant_w4g32_bf16(st, w, sc, bi, static_cast<uint16_t*>(buf(3)), ival(4), ival(5));
      }
    } else if (!w || !sc || (!bi && !q40) || !buf(3) || !buf(4) || !has_int(5) || !has_int(6) ||
               (kind == QuantKernel::QmvAdd && !buf(7))) {
      status = VPQ_ERR_NULL_POINTER;
    } else {
      const uint16_t* x = static_cast<const uint16_t*>(buf(3));
      uint16_t* y = static_cast<uint16_t*>(buf(4));
      const int K = ival(5), N = ival(6);
      const bool batched = kind == QuantKernel::QmvBatch || kind == QuantKernel::QmvBatchSwiglu ||
                           kind == QuantKernel::QmvBatchGeglu;          // rows = m_total in slot 7 (a missing one: 0 rows, refused)
      const int M = batched ? (has_int(7) ? ival(7) : 0) : (grid.x >= 32 ? static_cast<int>(grid.x / 32) : 1);
      const uint16_t* residual = kind == QuantKernel::QmvAdd ? static_cast<const uint16_t*>(buf(7)) : nullptr;
      const bool gather = kind == QuantKernel::GatherSwiglu || kind == QuantKernel::GatherGeglu ||
                          kind == QuantKernel::GatherDown;
      const bool grouped = kind == QuantKernel::GroupedSwiglu || kind == QuantKernel::GroupedGeglu ||
                           kind == QuantKernel::GroupedDown;
      if (fmt == QuantFormat::W8G64 && (kind == QuantKernel::Qmm || kind == QuantKernel::QmmSwiglu ||
                                        kind == QuantKernel::QmmGeglu)) {
        // gpu-kernels/metal/quant/affine_qmm_steel.metal:1601-1890: the 4-bit GEMM slots (7 = M, 8 = out_stride,
        // 9 = out_off for the strided gated form) over byte codes
        if (!has_int(7)) {
          status = VPQ_ERR_NULL_POINTER;
        } else {
          const int act = kind == QuantKernel::Qmm ? 0 : (kind == QuantKernel::QmmGeglu ? VPQ_GATE_GEGLU : VPQ_GATE_SWIGLU);
          status = vpq_qmm_gated_w8g64_bf16(st, w, sc, bi, x, y, K, N, ival(7), act != 0 && has_int(8) ? ival(8) : 0,
                                            act != 0 && has_int(9) ? ival(9) : 0, act);
        }
      } else if (fmt == QuantFormat::W4G64F16 && (kind == QuantKernel::Qmm || kind == QuantKernel::QmmSwiglu ||
                                                  kind == QuantKernel::QmmGeglu)) {
        // the fused GEMM of the binary16 build: slot 7 = M
        const int act = kind == QuantKernel::Qmm ? 0 : (kind == QuantKernel::QmmGeglu ? VPQ_GATE_GEGLU : VPQ_GATE_SWIGLU);
        status = !has_int(7) ? VPQ_ERR_NULL_POINTER : vpq_qmm_w4g64_f16(st, w, sc, bi, x, y, K, N, ival(7), act);
      } else if (fmt == QuantFormat::W4G32 && (kind == QuantKernel::Qmm || kind == QuantKernel::QmmGeglu)) {
        // gpu-kernels/metal/quant/affine_qmm_steel.metal:618-640, 1573-1596: slot 7 = M
        status = !has_int(7) ? VPQ_ERR_NULL_POINTER
                             : vpq_qmm_gated_w4g32_bf16(st, w, sc, bi, x, y, K, N, ival(7),
                                                        kind == QuantKernel::QmmGeglu ? VPQ_GATE_GEGLU : 0);
      } else if (fmt == QuantFormat::W8G64 && (kind == QuantKernel::SortedSwiglu || kind == QuantKernel::SortedDown)) {
        // gpu-kernels/metal/quant/affine_qmv.metal:2682-2719: slot 7 = srow, 8 = tile2e, one tile of two sorted
        // slots per grid.z; the expert count is the number of [N, K] byte slabs the bound code buffer holds
        if (!buf(7) || !buf(8)) {
          status = VPQ_ERR_NULL_POINTER;
        } else if (K <= 0 || N <= 0 || K % 64 != 0) {
          status = VPQ_ERR_BAD_SHAPE;
        } else {
          const std::size_t experts = _slots[0].bytes / (static_cast<std::size_t>(N) * static_cast<std::size_t>(K));
          const int E = experts > 0x7fffffffu ? 0x7fffffff : static_cast<int>(experts);
          const int npad = static_cast<int>(grid.z) * VPQ_QMV_GROUPED_SLOTS;
          const int32_t* srow = static_cast<const int32_t*>(buf(7));
          const int32_t* t2e = static_cast<const int32_t*>(buf(8));
          status = kind == QuantKernel::SortedDown
                       ? vpq_qmv_grouped_down_w8g64_bf16(st, w, sc, bi, x, y, K, N, npad, t2e, srow, E)
                       : vpq_qmv_grouped_gated_w8g64_bf16(st, w, sc, bi, x, y, K, N, npad, t2e, srow, E, VPQ_GATE_SWIGLU);
        }
      } else if (fmt == QuantFormat::W8G64 && grouped) {
        // :1069-1090, 1290-1366: slot 7 = npad, 8 = tile2e, 9 = srow / sdst, as the 4-bit grouped functions
        const bool down = kind == QuantKernel::GroupedDown;
        if (!has_int(7) || !buf(8) || !buf(9)) {
          status = VPQ_ERR_NULL_POINTER;
        } else if (K <= 0 || N <= 0 || K % 64 != 0) {
          status = VPQ_ERR_BAD_SHAPE;
        } else {
          const std::size_t experts = _slots[0].bytes / (static_cast<std::size_t>(N) * static_cast<std::size_t>(K));
          const int E = experts > 0x7fffffffu ? 0x7fffffff : static_cast<int>(experts);
          const std::size_t rows = down ? _slots[4].bytes / (static_cast<std::size_t>(N) * 2)
                                        : _slots[3].bytes / (static_cast<std::size_t>(K) * 2);
          const int nrows = rows > 0x7fffffffu ? 0x7fffffff : static_cast<int>(rows);
          const int32_t* t2e = static_cast<const int32_t*>(buf(8));
          const int32_t* idx = static_cast<const int32_t*>(buf(9));
          status = down ? vpq_qmm_grouped_down_w8g64_bf16(st, w, sc, bi, x, y, K, N, ival(7), t2e, idx, E, nrows)
                        : vpq_qmm_grouped_gated_w8g64_bf16(st, w, sc, bi, x, y, K, N, ival(7), t2e, idx, E, nrows,
                                                           kind == QuantKernel::GroupedGeglu ? VPQ_GATE_GEGLU
                                                                                             : VPQ_GATE_SWIGLU);
        }
      } else if (fmt == QuantFormat::W4G64F16) {
        if (kind == QuantKernel::QmvSwiglu || kind == QuantKernel::QmvGeglu || kind == QuantKernel::QmvBatchSwiglu ||
            kind == QuantKernel::QmvBatchGeglu) {
          const bool geglu = kind == QuantKernel::QmvGeglu || kind == QuantKernel::QmvBatchGeglu;
          status = vpq_qmv_gated_w4g64_f16(st, w, sc, bi, x, y, K, N, M, geglu ? VPQ_GATE_GEGLU : VPQ_GATE_SWIGLU);
        } else {
          status = vpq_qmv_w4g64_f16(st, w, sc, bi, x, y, K, N, M, residual);
        }
      } else if (fmt == QuantFormat::W8G64 && gather) {
        // gpu-kernels/metal/quant/affine_qmv.metal:962-990, 1295-1322, 1524-1552: slot 7 = pair_eid, 8 = top_k
        // (gate|up only), pairs = grid.z; the expert count is what the bound code buffer holds (K bytes a row)
        const bool down = kind == QuantKernel::GatherDown;
        if (!buf(7) || (!down && !has_int(8))) {
          status = VPQ_ERR_NULL_POINTER;
        } else if (K <= 0 || N <= 0 || K % 64 != 0) {
          status = VPQ_ERR_BAD_SHAPE;
        } else {
          const std::size_t experts = _slots[0].bytes / (static_cast<std::size_t>(N) * static_cast<std::size_t>(K));
          const int E = experts > 0x7fffffffu ? 0x7fffffff : static_cast<int>(experts);
          const int32_t* eid = static_cast<const int32_t*>(buf(7));
          const int npair = static_cast<int>(grid.z);
          status = down ? vpq_gather_down_qmv_w8g64_bf16(st, w, sc, bi, x, y, K, N, eid, npair, E)
                        : vpq_gather_qmv_gated_w8g64_bf16(st, w, sc, bi, x, y, K, N, eid, npair, ival(8), E,
                                                          kind == QuantKernel::GatherGeglu ? VPQ_GATE_GEGLU
                                                                                           : VPQ_GATE_SWIGLU);
        }
      } else if (fmt == QuantFormat::W8G64 && (kind == QuantKernel::QmvSwiglu || kind == QuantKernel::QmvGeglu)) {
        status = vpq_qmv_gated_w8g64_bf16(st, w, sc, bi, x, y, K, N, M,
                                          kind == QuantKernel::QmvGeglu ? VPQ_GATE_GEGLU : VPQ_GATE_SWIGLU);
      } else if (fmt == QuantFormat::W8G64) {
        status = vpq_qmv_w8g64_bf16(st, w, sc, bi, x, y, K, N, M, residual);
      } else if ((fmt == QuantFormat::W8G64F16 || fmt == QuantFormat::W8G32F16) && kind == QuantKernel::Qmm) {
        // the binary16 build's 8-bit GEMM, slot 7 = M: the dequant-once route on the binary16 dense GEMM
        uint16_t* w_deq = (in_scope || K <= 0 || N <= 0)
                              ? nullptr
                              : static_cast<uint16_t*>(s->qmv_workspace(static_cast<std::size_t>(N) * static_cast<std::size_t>(K) * 2));
        status = !has_int(7) ? VPQ_ERR_NULL_POINTER
                             : (w_deq == nullptr ? VPQ_ERR_WORKSPACE
                                                 : vpq_qmm_dense_route_w8_f16(st, fmt == QuantFormat::W8G64F16 ? 64 : 32, w, sc, bi, x,
                                                                              y, K, N, ival(7), w_deq, 1));
      } else if (fmt == QuantFormat::W8G32 && kind == QuantKernel::Qmm) {
        // gpu-kernels/metal/quant/affine_qmm_steel.metal:1674-1698, slot 7 = M: the dequant-once route, the
        // expansion in scratch of the stream (shared, so not inside a concurrent scope)
        uint16_t* w_deq = (in_scope || K <= 0 || N <= 0)
                              ? nullptr
                              : static_cast<uint16_t*>(s->qmv_workspace(static_cast<std::size_t>(N) * static_cast<std::size_t>(K) * 2));
        status = !has_int(7) ? VPQ_ERR_NULL_POINTER
                             : (w_deq == nullptr ? VPQ_ERR_WORKSPACE
                                                 : vpq_qmm_dense_route_w8g32_bf16(st, w, sc, bi, x, y, K, N, ival(7), w_deq, 1));
      } else if (fmt == QuantFormat::W8G32) {
        status = vpq_qmv_w8g32_bf16(st, w, sc, bi, x, y, K, N, M, residual);
      } else if (kind == QuantKernel::QmvGeglu || kind == QuantKernel::QmvBatchGeglu) {
        status = vpq_qmv_gated_w4g32_bf16(st, w, sc, q40 ? nullptr : bi, x, y, K, N, M, VPQ_GATE_GEGLU, q40 ? 1 : 0);
      } else {
        status = vpq_qmv_w4g32_bf16(st, w, sc, q40 ? nullptr : bi, x, y, K, N, M, residual, q40 ? 1 : 0);
      }
    }
  } else if (kind == QuantKernel::GatherSplit48 || kind == QuantKernel::GatherSplit84) {
    // gpu-kernels/metal/quant/affine_qmv.metal:1198-1260; the expert count is what the gate code buffer holds
    bool have = has_int(8) && has_int(9) && has_int(11) && buf(10);
    for (unsigned i = 0; i < 8; ++i) { have = have && buf(i); }
    if (!have) {
      status = VPQ_ERR_NULL_POINTER;
    } else if (ival(8) <= 0 || ival(8) % 64 != 0 || ival(9) <= 0) {
      status = VPQ_ERR_BAD_SHAPE;
    } else {
      const int K = ival(8), F = ival(9);
      const int gbits = kind == QuantKernel::GatherSplit48 ? 4 : 8, ubits = 12 - gbits;
      const std::size_t slab = static_cast<std::size_t>(F) * static_cast<std::size_t>(K) * gbits / 8;
      const std::size_t experts = _slots[0].bytes / slab;
      const int E = experts > 0x7fffffffu ? 0x7fffffff : static_cast<int>(experts);
      status = vpq_gather_qmv_gated_split_bf16(
          st, static_cast<const uint32_t*>(buf(0)), static_cast<const uint16_t*>(buf(1)), static_cast<const uint16_t*>(buf(2)),
          gbits, static_cast<const uint32_t*>(buf(3)), static_cast<const uint16_t*>(buf(4)),
          static_cast<const uint16_t*>(buf(5)), ubits, static_cast<const uint16_t*>(buf(6)), static_cast<uint16_t*>(buf(7)), K, F,
          static_cast<const int32_t*>(buf(10)), static_cast<int>(grid.z), ival(11), E, VPQ_GATE_SWIGLU);
    }
  } else if (kind == QuantKernel::Dequant) {
    // slots 0:w 1:scales 2:biases 3:w_deq 4:K 5:N
    if (!buf(0) || !buf(1) || !buf(2) || !buf(3) || !has_int(4) || !has_int(5)) {
      status = VPQ_ERR_NULL_POINTER;
    } else {
      status = vpq_dequant_w4g64_bf16(st, static_cast<const uint32_t*>(buf(0)), static_cast<const uint16_t*>(buf(1)),
                                      static_cast<const uint16_t*>(buf(2)), static_cast<uint16_t*>(buf(3)), ival(4), ival(5));
    }
  } else if (kind == QuantKernel::EmbedGather) {
    // gpu-kernels/metal/ops/llm_elementwise.metal:1676-1701: slots 0:ids 1:w 2:scales 3:biases 4:out 5:H,
    // grid (H, T, 1).  The table's row count is not a slot: it is what the code buffer holds.
    if (!buf(0) || !buf(1) || !buf(2) || !buf(3) || !buf(4) || !has_int(5)) {
      status = VPQ_ERR_NULL_POINTER;
    } else if (ival(5) <= 0 || ival(5) % 64 != 0) {
      status = VPQ_ERR_BAD_SHAPE;
    } else {
      const int H = ival(5);
      const std::size_t rows = _slots[1].bytes / (static_cast<std::size_t>(H) / 2);
      const int vocab = rows > 0x7fffffffu ? 0x7fffffff : static_cast<int>(rows);
      status = vpq_embed_gather_w4g64_bf16(st, static_cast<const int32_t*>(buf(0)), static_cast<const uint32_t*>(buf(1)),
                                           static_cast<const uint16_t*>(buf(2)), static_cast<const uint16_t*>(buf(3)),
                                           static_cast<uint16_t*>(buf(4)), H, static_cast<int>(grid.y), vocab);
    }
  } else if (kind == QuantKernel::Argmax || kind == QuantKernel::ArgmaxPartial || kind == QuantKernel::ArgmaxCombine) {
    // gpu-kernels/metal/ops/llm_elementwise.metal:2906-2941, 2977-3028, 3030-3062.  The partials of the
    // two-stage pair are two 4-byte slots per slab, as the reference's; only the pair reads them.
    if (kind == QuantKernel::Argmax) {
      status = (!buf(0) || !buf(1) || !has_int(2))
                   ? VPQ_ERR_NULL_POINTER
                   : vpq_argmax_bf16(st, static_cast<const uint16_t*>(buf(0)), static_cast<int32_t*>(buf(1)), ival(2), 1,
                                     nullptr, 0);
    } else if (kind == QuantKernel::ArgmaxPartial) {
      status = (!buf(0) || !buf(1) || !has_int(2) || !has_int(3))
                   ? VPQ_ERR_NULL_POINTER
                   : vpq_argmax_partial_bf16(st, static_cast<const uint16_t*>(buf(0)), static_cast<float*>(buf(1)), ival(2),
                                             ival(3));
    } else {
      status = (!buf(0) || !buf(1) || !has_int(2))
                   ? VPQ_ERR_NULL_POINTER
                   : vpq_argmax_combine(st, static_cast<const float*>(buf(0)), static_cast<int32_t*>(buf(1)), ival(2));
    }
  } else if (kind == QuantKernel::SampleTopp) {
    // gpu-kernels/metal/ops/llm_elementwise.metal:3116-3130: 0:logits 1:out_id 2:V 3:temp 4:top_p 5:seed 6:ws 7:n_iter
    // 8:rep 9:pres 10:top_k 11:min_p 12:seen
    bool have = buf(0) && buf(1) && buf(6) && buf(12);
    for (unsigned i : {2u, 3u, 4u, 5u, 7u, 8u, 9u, 10u, 11u}) { have = have && has_int(i); }
    auto fval = [&](unsigned i) { return _slots[i].fvalue; };
    status = !have ? VPQ_ERR_NULL_POINTER
                   : vpq_sample_topp_bf16(st, static_cast<const uint16_t*>(buf(0)), static_cast<int32_t*>(buf(1)), ival(2),
                                          fval(3), fval(4), static_cast<uint32_t>(_slots[5].ivalue), static_cast<uint16_t*>(buf(6)),
                                          ival(7), fval(8), fval(9), ival(10), fval(11), static_cast<uint8_t*>(buf(12)));
  } else if (kind == QuantKernel::QmvQkvRms) {
    // gpu-kernels/metal/quant/affine_qmv.metal:671-740: slots 0:w 1:scales 2:biases 3:x 4:norm_w 5:q_out 6:k_out 7:v_out
    // 8:K 9:q_rows 10:k_rows 11:v_rows 12:eps; the pack is the row-concatenated q|k|v
    if (!buf(0) || !buf(1) || !buf(2) || !buf(3) || !buf(4) || !buf(5) || !buf(6) || !has_int(8) || !has_int(9) ||
        !has_int(10) || !has_int(11) || !has_int(12) || (ival(11) > 0 && !buf(7))) {
      status = VPQ_ERR_NULL_POINTER;
    } else if (ival(8) <= 0 || ival(8) % 64 != 0 || ival(9) <= 0 || ival(10) <= 0 || ival(11) < 0) {
      status = VPQ_ERR_BAD_SHAPE;
    } else {
      const int K = ival(8);
      const int rows[3] = {ival(9), ival(10), ival(11)};
      const uint32_t* w[3];
      const uint16_t* sc[3];
      const uint16_t* bi[3];
      uint16_t* y[3] = {static_cast<uint16_t*>(buf(5)), static_cast<uint16_t*>(buf(6)), static_cast<uint16_t*>(buf(7))};
      const size_t row_words = (size_t)(fmt == QuantFormat::W8G64 ? K / 4 : K / 8);
      const size_t row_groups = (size_t)(fmt == QuantFormat::W4G32 ? K / 32 : K / 64);
      size_t r0 = 0;
      for (int i = 0; i < 3; ++i) {
        w[i] = static_cast<const uint32_t*>(buf(0)) + r0 * row_words;
        sc[i] = static_cast<const uint16_t*>(buf(1)) + r0 * row_groups;
        bi[i] = static_cast<const uint16_t*>(buf(2)) + r0 * row_groups;
        r0 += (size_t)rows[i];
      }
      // the normalized row: scratch of the stream (shared, so not inside a concurrent scope)
      uint16_t* xn = in_scope ? nullptr : static_cast<uint16_t*>(s->qmv_workspace((size_t)K * 2));
      const int format = fmt == QuantFormat::W8G64 ? VPQ_FORMAT_W8G64 : (fmt == QuantFormat::W4G32 ? VPQ_FORMAT_W4G32 : VPQ_FORMAT_W4G64);
      status = xn == nullptr ? VPQ_ERR_WORKSPACE
                             : vpq_qmv_qkv_rms_bf16(st, format, rows[2] > 0 ? 3 : 2, w, sc, bi, static_cast<const uint16_t*>(buf(3)),
                                                    static_cast<const uint16_t*>(buf(4)), y, K, rows, _slots[12].fvalue, xn);
    }
  } else if (kind == QuantKernel::QmvQkv) {
    // gpu-kernels/metal/quant/affine_qmv.metal:497-516: slots 0:w 1:scales 2:biases 3:x 4:q_out
    // 5:k_out 6:v_out 7:K 8:q_rows 9:k_rows 10:v_rows; the pack is the row-concatenated q|k|v.
    if (!buf(0) || !buf(1) || !buf(2) || !buf(3) || !buf(4) || !buf(5) || !has_int(7) || !has_int(8) || !has_int(9) ||
        !has_int(10) || (ival(10) > 0 && !buf(6))) {
      status = VPQ_ERR_NULL_POINTER;
    } else if (ival(7) <= 0 || ival(7) % 64 != 0 || ival(8) <= 0 || ival(9) <= 0 || ival(10) < 0) {
      status = VPQ_ERR_BAD_SHAPE;
    } else {
      const int K = ival(7);
      const int rows[3] = {ival(8), ival(9), ival(10)};
      const uint32_t* w[3];
      const uint16_t* sc[3];
      const uint16_t* bi[3];
      uint16_t* y[3] = {static_cast<uint16_t*>(buf(4)), static_cast<uint16_t*>(buf(5)), static_cast<uint16_t*>(buf(6))};
      // words of codes and groups per row of the format (:518-559: the 8-bit and the group-32 twins)
      const size_t row_words = (size_t)(fmt == QuantFormat::W8G64 ? K / 4 : K / 8);
      const size_t row_groups = (size_t)(fmt == QuantFormat::W4G32 ? K / 32 : K / 64);
      size_t r0 = 0;
      for (int i = 0; i < 3; ++i) {
        w[i] = static_cast<const uint32_t*>(buf(0)) + r0 * row_words;
        sc[i] = static_cast<const uint16_t*>(buf(1)) + r0 * row_groups;
        bi[i] = static_cast<const uint16_t*>(buf(2)) + r0 * row_groups;
        r0 += (size_t)rows[i];
      }
      const int count = rows[2] > 0 ? 3 : 2;
      const uint16_t* x = static_cast<const uint16_t*>(buf(3));
      if (fmt == QuantFormat::W4G64F16) {
        status = vpq_qmv_group_w4g64_f16(st, count, w, sc, bi, x, y, K, rows, 1);
      } else if (fmt == QuantFormat::W8G64) {
        status = vpq_qmv_group_w8g64_bf16(st, count, w, sc, bi, x, y, K, rows, 1);
      } else if (fmt == QuantFormat::W4G32) {
        status = vpq_qmv_group_w4g32_bf16(st, count, w, sc, bi, x, y, K, rows, 1, 0);
      } else {
        status = vpq_qmv_group_w4g64_bf16(st, count, w, sc, bi, x, y, K, rows, 1);
      }
    }
  } else {
    // slots 0:w 1:scales 2:biases 3:x 4:y 5:K 6:N, 7: residual | m_total | M
    if (!buf(0) || !buf(1) || !buf(2) || !buf(3) || !buf(4) || !has_int(5) || !has_int(6)) {
      status = VPQ_ERR_NULL_POINTER;
    } else {
      const uint32_t* w = static_cast<const uint32_t*>(buf(0));
      const uint16_t* sc = static_cast<const uint16_t*>(buf(1));
      const uint16_t* bi = static_cast<const uint16_t*>(buf(2));
      const uint16_t* x = static_cast<const uint16_t*>(buf(3));
      uint16_t* y = static_cast<uint16_t*>(buf(4));
      const int K = ival(5), N = ival(6);
      if (kind == QuantKernel::GatherSwiglu || kind == QuantKernel::GatherGeglu || kind == QuantKernel::GatherDown) {
        // gpu-kernels/metal/quant/affine_qmv.metal:928-960, 1265-1292, 1494-1522: slot 7 = pair_eid,
        // 8 = top_k (gate|up only), one (token, expert) pair per grid.z
        // (generative-models/qwen3/metal-qwen-model.cc:4190-4206).  The expert count is not a slot:
        // it is the number of [N, K/8] slabs the bound code buffer holds.
        const bool down = kind == QuantKernel::GatherDown;
        if (!buf(7) || (!down && !has_int(8))) {
          status = VPQ_ERR_NULL_POINTER;
        } else if (K <= 0 || N <= 0 || K % 64 != 0) {
          status = VPQ_ERR_BAD_SHAPE;
        } else {
          const std::size_t slab = static_cast<std::size_t>(N) * static_cast<std::size_t>(K / 2);
          const std::size_t experts = _slots[0].bytes / slab;
          const int E = experts > 0x7fffffffu ? 0x7fffffff : static_cast<int>(experts);
          const int npair = static_cast<int>(grid.z);
          const int32_t* eid = static_cast<const int32_t*>(buf(7));
          if (down) {
            status = vpq_gather_down_qmv_w4g64_bf16(st, w, sc, bi, x, y, K, N, eid, npair, E);
          } else {
            status = vpq_gather_qmv_gated_w4g64_bf16(st, w, sc, bi, x, y, K, N, eid, npair, ival(8), E,
                                                     kind == QuantKernel::GatherGeglu ? VPQ_GATE_GEGLU : VPQ_GATE_SWIGLU);
          }
        }
      } else if (kind == QuantKernel::SortedSwiglu || kind == QuantKernel::SortedDown) {
        // gpu-kernels/metal/quant/affine_qmv.metal:2682-2708: slot 7 = srow, 8 = tile2e, one tile of two sorted
        // slots per grid.z.  The expert count is the number of [N, K/8] slabs the bound code buffer holds.
        if (!buf(7) || !buf(8)) {
          status = VPQ_ERR_NULL_POINTER;
        } else if (K <= 0 || N <= 0 || K % 64 != 0) {
          status = VPQ_ERR_BAD_SHAPE;
        } else {
          const std::size_t slab = static_cast<std::size_t>(N) * static_cast<std::size_t>(K / 2);
          const std::size_t experts = _slots[0].bytes / slab;
          const int E = experts > 0x7fffffffu ? 0x7fffffff : static_cast<int>(experts);
          const int npad = static_cast<int>(grid.z) * VPQ_QMV_GROUPED_SLOTS;
          const int32_t* srow = static_cast<const int32_t*>(buf(7));
          const int32_t* t2e = static_cast<const int32_t*>(buf(8));
          status = kind == QuantKernel::SortedDown
                       ? vpq_qmv_grouped_down_w4g64_bf16(st, w, sc, bi, x, y, K, N, npad, t2e, srow, E)
                       : vpq_qmv_grouped_gated_w4g64_bf16(st, w, sc, bi, x, y, K, N, npad, t2e, srow, E, VPQ_GATE_SWIGLU);
        }
      } else if (kind == QuantKernel::GroupedSwiglu || kind == QuantKernel::GroupedGeglu ||
                 kind == QuantKernel::GroupedDown) {
        // gpu-kernels/metal/quant/affine_qmm_steel.metal:1042-1066, 1266-1339: slot 7 = npad (sorted slots,
        // whole blocks of vpq_qmm_grouped_block_rows()), 8 = tile2e, 9 = srow (gate|up) or sdst (down)
        // (generative-models/qwen3/metal-qwen-model.cc:4239-4264).  Expert count and the row counts the
        // index buffers may name are what the bound buffers hold.
        const bool down = kind == QuantKernel::GroupedDown;
        if (!has_int(7) || !buf(8) || !buf(9)) {
          status = VPQ_ERR_NULL_POINTER;
        } else if (K <= 0 || N <= 0 || K % 64 != 0) {
          status = VPQ_ERR_BAD_SHAPE;
        } else {
          const std::size_t slab = static_cast<std::size_t>(N) * static_cast<std::size_t>(K / 2);
          const std::size_t experts = _slots[0].bytes / slab;
          const int E = experts > 0x7fffffffu ? 0x7fffffff : static_cast<int>(experts);
          const std::size_t rows = down ? _slots[4].bytes / (static_cast<std::size_t>(N) * 2)
                                        : _slots[3].bytes / (static_cast<std::size_t>(K) * 2);
          const int nrows = rows > 0x7fffffffu ? 0x7fffffff : static_cast<int>(rows);
          const int32_t* t2e = static_cast<const int32_t*>(buf(8));
          const int32_t* idx = static_cast<const int32_t*>(buf(9));
          if (down) {
            status = vpq_qmm_grouped_down_w4g64_bf16(st, w, sc, bi, x, y, K, N, ival(7), t2e, idx, E, nrows);
          } else {
            status = vpq_qmm_grouped_gated_w4g64_bf16(st, w, sc, bi, x, y, K, N, ival(7), t2e, idx, E, nrows,
                                                      kind == QuantKernel::GroupedGeglu ? VPQ_GATE_GEGLU : VPQ_GATE_SWIGLU);
          }
        }
      } else if (kind == QuantKernel::Qmm) {
        if (!has_int(7)) {
          status = VPQ_ERR_NULL_POINTER;
        } else {
          status = vpq_qmm_w4g64_bf16(st, w, sc, bi, x, y, K, N, ival(7), nullptr, nullptr, 0, 0.f, nullptr);
        }
      } else if (kind == QuantKernel::QmmSwiglu || kind == QuantKernel::QmmGeglu) {
        // gpu-kernels/metal/quant/affine_qmm_steel.metal:801-947: slot 7 = M; the strided twin adds
        // 8 = out_stride, 9 = out_off.  Rows go to the GEMV arithmetic when there are at most 16,
        // the choice the reference makes at its call sites.
        if (!has_int(7)) {
          status = VPQ_ERR_NULL_POINTER;
        } else {
          const int stride = has_int(8) ? ival(8) : 0, off = has_int(9) ? ival(9) : 0;
          status = vpq_qmm_gated_w4g64_bf16(st, w, sc, bi, x, y, K, N, ival(7), stride, off,
                                            kind == QuantKernel::QmmGeglu ? VPQ_GATE_GEGLU : VPQ_GATE_SWIGLU);
        }
      } else if (kind == QuantKernel::QmvGeluMul) {
        // gpu-kernels/metal/quant/affine_qmv.metal:751-768: slot 7 = the multiplier
        const uint16_t* mul = static_cast<const uint16_t*>(buf(7));
        status = mul == nullptr ? VPQ_ERR_NULL_POINTER : vpq_qmv_gelu_mul_w4g64_bf16(st, w, sc, bi, x, y, K, N, mul);
      } else if (kind == QuantKernel::QmvSwiglu || kind == QuantKernel::QmvGeglu || kind == QuantKernel::QmvBatchSwiglu ||
                 kind == QuantKernel::QmvBatchGeglu) {
        // gpu-kernels/metal/quant/affine_qmv.metal:891-906: N = 2*ffn, rows from grid.x; the batched forms
        // (:2336-2354, 2854-2872, 3003) carry m_total in slot 7
        const bool batched = kind == QuantKernel::QmvBatchSwiglu || kind == QuantKernel::QmvBatchGeglu;
        const int M = batched ? (has_int(7) ? ival(7) : 0) : (grid.x >= 32 ? static_cast<int>(grid.x / 32) : 1);
        const bool geglu = kind == QuantKernel::QmvGeglu || kind == QuantKernel::QmvBatchGeglu;
        status = vpq_qmv_gated_w4g64_bf16(st, w, sc, bi, x, y, K, N, M, VPQ_QMV_AUTO, geglu ? VPQ_GATE_GEGLU : VPQ_GATE_SWIGLU);
      } else {
        int M = 1;
        const uint16_t* residual = nullptr;
        if (kind == QuantKernel::Qmv) {
          M = grid.x >= 32 ? static_cast<int>(grid.x / 32) : 1;
        } else if (kind == QuantKernel::QmvAdd) {
          M = grid.x >= 32 ? static_cast<int>(grid.x / 32) : 1;
          residual = static_cast<const uint16_t*>(buf(7));
          if (residual == nullptr) { status = VPQ_ERR_NULL_POINTER; }
        } else {
          if (!has_int(7)) { status = VPQ_ERR_NULL_POINTER; }
          M = ival(7);
        }
        if (status == VPQ_OK) {
          // The split-K scratch is shared by the stream, so concurrent dispatches go without it.
          void* ws = nullptr;
          std::size_t ws_bytes = 0;
          if (!in_scope && K > 0 && N > 0 && M > 0 && M <= 16) {
            ws_bytes = vpq_qmv_workspace_bytes(K, N, M);
            ws = s->qmv_workspace(ws_bytes);
            if (ws == nullptr) { ws_bytes = 0; }
          }
          status = vpq_qmv_w4g64_bf16(st, w, sc, bi, x, y, K, N, M, residual, ws, ws_bytes, VPQ_QMV_AUTO);
        }
      }
    }
  }
  if (status != VPQ_OK) { s->record_error(status, _fn.name()); }
  ++_n_dispatch;
}

// ---------------------------------------------------------------- QuantLinear
void quant_linear_forward(CommandStream& stream, const Linear& lin, const DeviceBuffer& x, std::size_t x_off,
                          const DeviceBuffer& y, std::size_t y_off, int M, const LoraFactors* lora,
                          const DeviceBuffer* lora_t)
{
  if (!stream.valid()) { return; }
  if (lin.codes == nullptr || lin.scales == nullptr || lin.qbias == nullptr || lin.codes->empty() ||
      lin.scales->empty() || lin.qbias->empty() || x.empty() || y.empty()) {
    stream.record_error(VPQ_ERR_NULL_POINTER, "quant_linear_forward");
    return;
  }
  const uint32_t* w = reinterpret_cast<const uint32_t*>(static_cast<const char*>(lin.codes->data()) + lin.codes_off);
  const uint16_t* sc = reinterpret_cast<const uint16_t*>(static_cast<const char*>(lin.scales->data()) + lin.scales_off);
  const uint16_t* bi = reinterpret_cast<const uint16_t*>(static_cast<const char*>(lin.qbias->data()) + lin.qbias_off);
  const uint16_t* xp = reinterpret_cast<const uint16_t*>(static_cast<const char*>(x.data()) + x_off);
  uint16_t* yp = reinterpret_cast<uint16_t*>(static_cast<char*>(y.data()) + y_off);
  hipStream_t st = static_cast<hipStream_t>(stream.native());
  int status;
  const bool with_lora = lora != nullptr && lora->a != nullptr && lora->b != nullptr && lora->rank > 0 &&
                         lora->strength != 0.f && !lora->a->empty() && !lora->b->empty();
  const bool w4g64 = lin.bits == 4 && lin.group == 64;
  if (!w4g64) {
    // The format twins: their own size-based entrances; an adapter goes by the dequant-once route (their fused
    // kernels take none), the expansion in scratch of the stream.
    if (!((lin.bits == 8 || lin.bits == 4) && (lin.group == 64 || lin.group == 32))) {
      stream.record_error(VPQ_ERR_BAD_SHAPE, "quant_linear_forward: pack format");
      return;
    }
    if (with_lora) {
      if (lora_t == nullptr || lora_t->size() < static_cast<std::size_t>(M) * lora->rank * 2) {
        stream.record_error(VPQ_ERR_WORKSPACE, "quant_linear_forward: lora_t scratch too small");
        return;
      }
      const int format = lin.bits == 8 ? (lin.group == 64 ? VPQ_FORMAT_W8G64 : VPQ_FORMAT_W8G32) : VPQ_FORMAT_W4G32;
      uint16_t* w_deq = static_cast<uint16_t*>(stream.qmv_workspace((size_t)lin.N * (size_t)lin.K * 2));
      status = w_deq == nullptr
                   ? VPQ_ERR_WORKSPACE
                   : vpq_qmm_dense_route_lora_bf16(st, format, w, sc, bi, xp, yp, lin.K, lin.N, M, w_deq, 1,
                                                   static_cast<const uint16_t*>(lora->a->data()),
                                                   static_cast<const uint16_t*>(lora->b->data()), lora->rank,
                                                   lora->strength, static_cast<uint16_t*>(lora_t->data()));
    } else if (lin.bits == 8 && lin.group == 32) {
      // 8-bit codes in groups of 32: the GEMV in slabs of 16 rows up to 64 rows, the dequant-once route above (its
      // expansion in scratch of the stream), which is the route the reference's codec takes for this format
      status = VPQ_OK;
      if (M <= 64) {
        for (int m0 = 0; m0 < M && status == VPQ_OK; m0 += 16) {
          const int rows = M - m0 < 16 ? M - m0 : 16;
          status = vpq_qmv_w8g32_bf16(st, w, sc, bi, xp + (size_t)m0 * lin.K, yp + (size_t)m0 * lin.N, lin.K, lin.N, rows, nullptr);
        }
      } else {
        uint16_t* w_deq = static_cast<uint16_t*>(stream.qmv_workspace((size_t)lin.N * (size_t)lin.K * 2));
        status = w_deq == nullptr ? VPQ_ERR_WORKSPACE
                                  : vpq_qmm_dense_route_w8g32_bf16(st, w, sc, bi, xp, yp, lin.K, lin.N, M, w_deq, 1);
      }
    } else {
      status = lin.bits == 8 ? vpq_linear_w8g64_bf16(st, w, sc, bi, xp, yp, lin.K, lin.N, M)
                             : vpq_linear_w4g32_bf16(st, w, sc, bi, xp, yp, lin.K, lin.N, M);
    }
  } else if (with_lora) {
    // An adapter always takes the GEMM route: its second factor is folded into the tile's accumulator.
    if (lora_t == nullptr || lora_t->size() < static_cast<std::size_t>(M) * lora->rank * 2) {
      stream.record_error(VPQ_ERR_WORKSPACE, "quant_linear_forward: lora_t scratch too small");
      return;
    }
    status = vpq_qmm_w4g64_bf16(st, w, sc, bi, xp, yp, lin.K, lin.N, M, static_cast<const uint16_t*>(lora->a->data()),
                                static_cast<const uint16_t*>(lora->b->data()), lora->rank, lora->strength,
                                static_cast<uint16_t*>(lora_t->data()));
  } else {
    void* ws = nullptr;
    std::size_t ws_bytes = 0;
    if (M <= 16 && M > 0 && lin.K > 0 && lin.N > 0) {
      ws_bytes = vpq_qmv_workspace_bytes(lin.K, lin.N, M);
      ws = stream.qmv_workspace(ws_bytes);
      if (ws == nullptr) { ws_bytes = 0; }
    }
    status = vpq_linear_w4g64_bf16(st, w, sc, bi, xp, yp, lin.K, lin.N, M, ws, ws_bytes);
  }
  if (status != VPQ_OK) { stream.record_error(status, "quant_linear_forward"); }
}

}  // namespace vpipe_amd

// Torch op registration layer: defines the reference's Marlin op schemas in the
// `_C` and `_moe_C` namespaces and forwards them to the C ABI of
// libsonar_marlin.so.  No kernels live here.
//
// Schemas follow csrc/libtorch_stable/torch_bindings.cpp:96-115 and
// csrc/libtorch_stable/moe/torch_bindings.cpp:76-89 of the reference;
// argument checks follow marlin.cu:626-882, gptq_marlin_repack.cu:289-317,
// awq_marlin_repack.cu:231-254 and moe/marlin_moe_wna16/ops.cu:630-879.
//
// The repack ops return the Marlin tile order bit for bit, because that is
// what every caller stores.  The gfx950 kernels stream a different order, so
// the GEMM ops convert a weight tensor the first time they see it and keep the
// converted copy, keyed by the tensor's address.  An entry is valid for one
// (address, tensor object, shape, version counter).  What invalidates it:
//   * the repack ops drop every entry whose source memory overlaps the tensor
//     they have just written (a reload through `x.data = ops.gptq_marlin_repack(...)`
//     is safe even when the allocator hands the old address back);
//   * a miss drops every entry of the same tensor object at another address
//     (`x.data = ...` keeps the object) and every entry whose tensor is gone;
//   * an in-place op on the tensor itself bumps its version counter;
//   * marlin_weight_cache_invalidate(tensor) / marlin_weight_cache_clear().
// What nothing here can see: bytes rewritten in place through another view
// (`x.data.copy_(...)`, any write to an inference-mode tensor).  After such a
// write the caller must call marlin_weight_cache_invalidate on the tensor.
// A miss while the stream is being captured into a graph is an error (the
// conversion would be recorded instead of run): warm every weight up before
// capture.  The conversion runs on the calling stream; a hit from another
// stream waits for it through an event.
#include <ATen/ATen.h>
#include <hip/hip_runtime_api.h>
#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <algorithm>
#include <iterator>
#include <mutex>
#include <optional>
#include <tuple>
#include <unordered_map>

#include "sonar_marlin.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

void raise_if_failed(int rc) {
  if (rc == SONAR_OK) return;
  const char* msg = sonar_marlin_last_error();
  if (rc == SONAR_E_UNSUPPORTED) {
    TORCH_CHECK_NOT_IMPLEMENTED(false, msg);
  }
  TORCH_CHECK(false, msg);
}

void* current_stream(const Tensor& t) {
  return (void*)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.get_device()).stream();
}

int dtype_code(const Tensor& a) {
  if (a.scalar_type() == at::kHalf) return SONAR_DTYPE_F16;
  if (a.scalar_type() == at::kBFloat16) return SONAR_DTYPE_BF16;
  TORCH_CHECK_NOT_IMPLEMENTED(
      false, "unsupported `a` scalar_type: only float16 / bfloat16 activations (W4A16) are built");
  return -1;
}

// ---------------------------------------------------------------- weight cache
struct NativeEntry {
  c10::weak_intrusive_ptr<c10::TensorImpl> source;   // the Marlin tensor, not kept alive by the cache
  Tensor native;
  int64_t size_k, size_n, experts;
  uint32_t version;
  size_t source_bytes;
  hipStream_t stream;    // the stream the conversion ran on
  hipEvent_t ready;      // recorded behind the conversion; null once it is known to have finished
};

std::mutex g_cache_mutex;
std::unordered_map<const void*, NativeEntry> g_cache;

uint32_t version_of(const Tensor& t) { return t.is_inference() ? 0u : t._version(); }

void drop_event(NativeEntry& e) {
  if (e.ready != nullptr) (void)hipEventDestroy(e.ready);
  e.ready = nullptr;
}

// Refuses a conversion while `stream` is being captured: the conversion kernels would be
// recorded into the graph instead of run, and the cached copy would be read before it exists.
void refuse_during_capture(hipStream_t stream, const char* what) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  TORCH_CHECK(status == hipStreamCaptureStatusNone, what,
              " has not been used before and the stream is being captured into a graph: its one-time "
              "conversion to the gfx950 streaming order cannot run inside a capture.  Call the op once on "
              "every weight (a warm-up step) before capturing.");
}

// A hit from another stream than the one that converted must not overtake the conversion.
// While `stream` is being captured nothing is asked of the event (event queries and waits on
// events from outside the capture invalidate it): a capture starts behind a device-wide
// synchronisation, so the conversion has finished.
void wait_for_conversion(NativeEntry& e, hipStream_t stream) {
  if (e.ready == nullptr) return;
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) (void)hipGetLastError();
  if (status != hipStreamCaptureStatusNone) return;
  if (hipEventQuery(e.ready) == hipSuccess) {
    drop_event(e);
    return;
  }
  (void)hipGetLastError();   // hipErrorNotReady
  if (stream != e.stream) (void)hipStreamWaitEvent(stream, e.ready, 0);
}

// Drops every entry whose source bytes overlap [begin, begin + bytes).
void invalidate_range_locked(const void* begin, size_t bytes) {
  const char* lo = static_cast<const char*>(begin);
  const char* hi = lo + bytes;
  for (auto it = g_cache.begin(); it != g_cache.end();) {
    const char* s = static_cast<const char*>(it->first);
    if (s < hi && lo < s + it->second.source_bytes) {
      drop_event(it->second);
      it = g_cache.erase(it);
    } else {
      ++it;
    }
  }
}

void record_conversion(NativeEntry& e, hipStream_t stream) {
  e.stream = stream;
  e.ready = nullptr;
  if (hipEventCreateWithFlags(&e.ready, hipEventDisableTiming) != hipSuccess || hipEventRecord(e.ready, stream) != hipSuccess) {
    (void)hipGetLastError();
    drop_event(e);
  }
}

// Before a new entry for `t` goes in: entries of tensors that are gone, and entries of this
// tensor object at another address (`x.data = ...` keeps the object alive), leave.
void evict_stale_locked(const Tensor& t, const void* key) {
  for (auto it = g_cache.begin(); it != g_cache.end();) {
    const bool gone = it->second.source.expired();
    const bool moved = !gone && it->first != key && it->second.source._unsafe_get_target() == t.unsafeGetTensorImpl();
    if (gone || moved) {
      drop_event(it->second);
      it = g_cache.erase(it);
    } else {
      ++it;
    }
  }
}

// b_q_weight: (K/16, 2N) or (E, K/16, 2N) int32 in Marlin order; (K/16, 4N) for 8-bit codes.
// `a8`: the 4-bit order of 8-bit activations (32 x 32 tiles).
Tensor native_weights(const Tensor& b_q_weight, int64_t size_k, int64_t size_n, int64_t experts, int bits = 4,
                      bool a8 = false) {
  const void* key = b_q_weight.const_data_ptr();
  hipStream_t stream = (hipStream_t)current_stream(b_q_weight);
  const int64_t key_k = a8 ? -1000 - size_k : size_k;   // the cache entry says which order it was converted from
  {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_cache.find(key);
    if (it != g_cache.end() && !it->second.source.expired() &&
        it->second.source._unsafe_get_target() == b_q_weight.unsafeGetTensorImpl() &&
        it->second.size_k == key_k && it->second.size_n == size_n && it->second.experts == experts &&
        it->second.version == version_of(b_q_weight)) {
      wait_for_conversion(it->second, stream);
      return it->second.native;
    }
  }
  refuse_during_capture(stream, "This weight tensor");
  Tensor native = at::empty_like(b_q_weight);
  const int64_t words = size_k * size_n / (32 / bits);
  const uint32_t* src = static_cast<const uint32_t*>(b_q_weight.const_data_ptr());
  uint32_t* dst = static_cast<uint32_t*>(native.mutable_data_ptr());
  for (int64_t e = 0; e < experts; ++e)
    raise_if_failed(a8        ? sonar_marlin_a8_to_gfx950(src + e * words, dst + e * words, size_k, size_n,
                                                          current_stream(b_q_weight))
                    : bits == 8 ? sonar_marlin8_to_gfx950(src + e * words, dst + e * words, size_k, size_n,
                                                          current_stream(b_q_weight))
                                : sonar_marlin_to_gfx950(src + e * words, dst + e * words, size_k, size_n,
                                                         current_stream(b_q_weight)));
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  evict_stale_locked(b_q_weight, key);
  invalidate_range_locked(key, b_q_weight.nbytes());
  NativeEntry entry{c10::weak_intrusive_ptr<c10::TensorImpl>(b_q_weight.getIntrusivePtr()), native, key_k, size_n,
                    experts, version_of(b_q_weight), b_q_weight.nbytes(), stream, nullptr};
  record_conversion(entry, stream);
  g_cache.insert_or_assign(key, entry);
  return native;
}

// MXFP4 block scales as the reference's callers pass them (float8_e8m0fnu exponent
// bytes in marlin_permute_scales order with every four neighbours in the order
// 0, 2, 1, 3; marlin_utils_fp4.py:123-135) -> bfloat16 powers of two in plain
// marlin_permute_scales order, which the kernels read.  Cached like the weights.
// `exponent_offset` is added to every exponent: 0 for MXFP4, 120 for MXFP8, whose
// kernels expect the scales times 2^120 (the fp8 codes are read as bf16 numbers
// with the same exponent field); exponents past the bf16 range become infinity.
Tensor mx_scales_as_bf16(const Tensor& b_scales, int64_t exponent_offset) {
  const void* key = b_scales.const_data_ptr();
  hipStream_t stream = (hipStream_t)current_stream(b_scales);
  {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_cache.find(key);
    if (it != g_cache.end() && !it->second.source.expired() &&
        it->second.source._unsafe_get_target() == b_scales.unsafeGetTensorImpl() && it->second.size_k == -1 &&
        it->second.size_n == exponent_offset && it->second.version == version_of(b_scales)) {
      wait_for_conversion(it->second, stream);
      return it->second.native;
    }
  }
  refuse_during_capture(stream, "This tensor of float8_e8m0fnu block scales");
  TORCH_CHECK(b_scales.numel() % 4 == 0, "b_scales.numel() must be a multiple of 4");
  const Tensor bytes = b_scales.view(at::kByte);
  const Tensor order = at::tensor({0, 2, 1, 3}, at::TensorOptions().dtype(at::kLong).device(b_scales.device()));
  const Tensor e = bytes.reshape({-1, 4}).index_select(1, order).reshape(bytes.sizes()).to(at::kShort) +
                   exponent_offset;
  // bfloat16 2^(e - 127): exponent field e; e = 0 is the subnormal 2^-127
  const Tensor bits = at::where(e == 0, at::full_like(e, 0x40), at::clamp_max(e, 255) * 128);
  Tensor out = bits.view(at::kBFloat16);
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  evict_stale_locked(b_scales, key);
  invalidate_range_locked(key, b_scales.nbytes());
  NativeEntry entry{c10::weak_intrusive_ptr<c10::TensorImpl>(b_scales.getIntrusivePtr()), out, -1, exponent_offset,
                    -1, version_of(b_scales), b_scales.nbytes(), stream, nullptr};
  record_conversion(entry, stream);
  g_cache.insert_or_assign(key, entry);
  return out;
}

// NVFP4 block scales as the reference's callers pass them (bytes of the special 8-bit format
// of nvfp4_marlin_process_scales, in marlin_permute_scales order with every four neighbours in
// the order 0, 2, 1, 3; marlin_utils_fp4.py:61-120) -> numbers of the activation type in plain
// marlin_permute_scales order, which the kernels read: a byte b stands for the half-precision
// number with the bits b << 7 (dequant.h:520-549), and the dequantised code of the reference
// carries 2^-14 (half) or 2^-126 (bfloat16), which is folded in here.  Cached like the weights.
Tensor nvfp4_scales_as_16bit(const Tensor& b_scales, at::ScalarType a_type) {
  const void* key = b_scales.const_data_ptr();
  const int64_t tag = a_type == at::kHalf ? -16 : -17;   // stored in size_n: which conversion this entry holds
  hipStream_t stream = (hipStream_t)current_stream(b_scales);
  {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_cache.find(key);
    if (it != g_cache.end() && !it->second.source.expired() &&
        it->second.source._unsafe_get_target() == b_scales.unsafeGetTensorImpl() && it->second.size_k == -1 &&
        it->second.size_n == tag && it->second.version == version_of(b_scales)) {
      wait_for_conversion(it->second, stream);
      return it->second.native;
    }
  }
  refuse_during_capture(stream, "This tensor of float8_e4m3fn block scales");
  TORCH_CHECK(b_scales.numel() % 4 == 0, "b_scales.numel() must be a multiple of 4");
  const Tensor bytes = b_scales.view(at::kByte);
  const Tensor order = at::tensor({0, 2, 1, 3}, at::TensorOptions().dtype(at::kLong).device(b_scales.device()));
  const Tensor plain = bytes.reshape({-1, 4}).index_select(1, order).reshape(bytes.sizes());
  const Tensor as_half = (plain.to(at::kShort) * 128).view(at::kHalf);   // the bits b << 7
  Tensor out = (as_half.to(at::kFloat) * (a_type == at::kHalf ? 0x1p-14 : 0x1p-126)).to(a_type);
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  evict_stale_locked(b_scales, key);
  invalidate_range_locked(key, b_scales.nbytes());
  NativeEntry entry{c10::weak_intrusive_ptr<c10::TensorImpl>(b_scales.getIntrusivePtr()), out, -1, tag,
                    -1, version_of(b_scales), b_scales.nbytes(), stream, nullptr};
  record_conversion(entry, stream);
  g_cache.insert_or_assign(key, entry);
  return out;
}

bool is_mx_scale_type(const Tensor& t) {
  return t.scalar_type() == at::kFloat8_e8m0fnu || t.scalar_type() == at::kByte;
}

int64_t marlin_weight_cache_clear() {
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  const int64_t n = (int64_t)g_cache.size();
  for (auto& kv : g_cache) drop_event(kv.second);
  g_cache.clear();
  return n;
}

// Drops the converted copies made from the memory of `t` (weights or block scales): to be called
// after the bytes of `t` were rewritten in place in a way that leaves its version counter alone.
int64_t marlin_weight_cache_invalidate(const Tensor& t) {
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  const size_t before = g_cache.size();
  if (t.defined() && t.numel() > 0) invalidate_range_locked(t.const_data_ptr(), t.nbytes());
  return (int64_t)(before - g_cache.size());
}

// The repack ops have just written `out`: whatever was converted from that memory before is stale.
void forget_memory_of(const Tensor& out) {
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  if (out.numel() > 0) invalidate_range_locked(out.const_data_ptr(), out.nbytes());
}

const void* opt_ptr(const OptTensor& t) {
  return (t.has_value() && t->numel() > 0) ? t->const_data_ptr() : nullptr;
}

// ---------------------------------------------------------------- repack
Tensor gptq_marlin_repack(const Tensor& b_q_weight, const Tensor& perm, int64_t size_k,
                          int64_t size_n, int64_t num_bits, bool is_a_8bit) {
  TORCH_CHECK(num_bits == 4 || num_bits == 8, "num_bits must be 4 or 8. Got = ", num_bits);
  const int64_t pack_factor = 32 / num_bits;
  TORCH_CHECK(size_k % 16 == 0, "size_k = ", size_k, " is not divisible by tile_k_size = ", 16);
  TORCH_CHECK(size_n % 64 == 0, "size_n = ", size_n, " is not divisible by tile_n_size = ", 64);
  TORCH_CHECK(b_q_weight.dim() == 2 && b_q_weight.size(0) == size_k / pack_factor,
              "Shape mismatch: b_q_weight.size(0) = ", b_q_weight.size(0), ", size_k = ", size_k,
              ", pack_factor = ", pack_factor);
  TORCH_CHECK(b_q_weight.size(1) == size_n, "b_q_weight.size(1) = ", b_q_weight.size(1),
              " is not size_n = ", size_n);
  TORCH_CHECK(b_q_weight.is_cuda(), "b_q_weight is not on GPU");
  TORCH_CHECK(b_q_weight.is_contiguous(), "b_q_weight is not contiguous");
  TORCH_CHECK(b_q_weight.scalar_type() == at::kInt, "b_q_weight type is not kInt");
  TORCH_CHECK(perm.is_cuda(), "perm is not on GPU");
  TORCH_CHECK(perm.is_contiguous(), "perm is not contiguous");
  TORCH_CHECK(perm.scalar_type() == at::kInt, "perm type is not at::kInt");
  const bool has_perm = perm.numel() > 0;
  TORCH_CHECK(!has_perm || perm.numel() == size_k, "perm.numel() = ", perm.numel(),
              " is not size_k = ", size_k);

  c10::hip::HIPGuardMasqueradingAsCUDA guard(b_q_weight.device());
  Tensor out = at::empty({size_k / 16, size_n * 16 / pack_factor}, b_q_weight.options());
  if (is_a_8bit) {
    // gptq_marlin_repack.cu:147 (static_assert(!is_a_8bit) under has_perm), :354-357
    TORCH_CHECK(!has_perm, "Unsupported repack config: num_bits = ", num_bits, ", has_perm = ", has_perm,
                ", is_a_8bit = ", is_a_8bit);
    raise_if_failed(sonar_gptq_marlin_repack_a8(static_cast<const uint32_t*>(b_q_weight.const_data_ptr()),
                                                static_cast<uint32_t*>(out.mutable_data_ptr()), size_k, size_n,
                                                (int)num_bits, current_stream(b_q_weight)));
    forget_memory_of(out);
    return out;
  }
  raise_if_failed(sonar_gptq_marlin_repack(
      static_cast<const uint32_t*>(b_q_weight.const_data_ptr()),
      has_perm ? static_cast<const int32_t*>(perm.const_data_ptr()) : nullptr,
      static_cast<uint32_t*>(out.mutable_data_ptr()), size_k, size_n, (int)num_bits,
      current_stream(b_q_weight)));
  forget_memory_of(out);
  return out;
}

Tensor awq_marlin_repack(const Tensor& b_q_weight, int64_t size_k, int64_t size_n, int64_t num_bits,
                         bool is_a_8bit) {
  TORCH_CHECK(num_bits == 4 || num_bits == 8, "num_bits must be 4 or 8. Got = ", num_bits);
  const int64_t pack_factor = 32 / num_bits;
  TORCH_CHECK(size_k % 16 == 0, "size_k = ", size_k, " is not divisible by tile_k_size = ", 16);
  TORCH_CHECK(size_n % 64 == 0, "size_n = ", size_n, " is not divisible by tile_n_size = ", 64);
  TORCH_CHECK(b_q_weight.dim() == 2 && b_q_weight.size(0) == size_k,
              "b_q_weight.size(0) = ", b_q_weight.size(0), " is not size_k = ", size_k);
  TORCH_CHECK(b_q_weight.size(1) == size_n / pack_factor, "Shape mismatch: b_q_weight.size(1) = ",
              b_q_weight.size(1), ", size_n = ", size_n, ", pack_factor = ", pack_factor);
  TORCH_CHECK(b_q_weight.is_cuda(), "b_q_weight is not on GPU");
  TORCH_CHECK(b_q_weight.is_contiguous(), "b_q_weight is not contiguous");
  TORCH_CHECK(b_q_weight.scalar_type() == at::kInt, "b_q_weight type is not kInt");

  c10::hip::HIPGuardMasqueradingAsCUDA guard(b_q_weight.device());
  Tensor out = at::empty({size_k / 16, size_n * 16 / pack_factor}, b_q_weight.options());
  raise_if_failed((is_a_8bit ? sonar_awq_marlin_repack_a8 : sonar_awq_marlin_repack)(
      static_cast<const uint32_t*>(b_q_weight.const_data_ptr()), static_cast<uint32_t*>(out.mutable_data_ptr()),
      size_k, size_n, (int)num_bits, current_stream(b_q_weight)));
  forget_memory_of(out);
  return out;
}

Tensor marlin_to_gfx950(const Tensor& b_q_weight, int64_t size_k, int64_t size_n) {
  TORCH_CHECK(b_q_weight.is_cuda() && b_q_weight.is_contiguous() && b_q_weight.scalar_type() == at::kInt,
              "b_q_weight must be a contiguous int32 GPU tensor");
  TORCH_CHECK(b_q_weight.numel() == size_k * size_n / 8, "b_q_weight has ", b_q_weight.numel(),
              " words, expected ", size_k * size_n / 8);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(b_q_weight.device());
  Tensor out = at::empty_like(b_q_weight);
  raise_if_failed(sonar_marlin_to_gfx950(static_cast<const uint32_t*>(b_q_weight.const_data_ptr()),
                                         static_cast<uint32_t*>(out.mutable_data_ptr()), size_k, size_n,
                                         current_stream(b_q_weight)));
  return out;
}

// marlin_int4_fp8_preprocess.cu:68-117
Tensor marlin_int4_fp8_preprocess(const Tensor& qweight, const OptTensor& qzeros_or_none, bool inplace) {
  TORCH_CHECK(qweight.is_cuda(), "qweight is not on GPU");
  TORCH_CHECK(qweight.scalar_type() == at::kInt, "qweight.dtype != torch.int32");
  TORCH_CHECK(qweight.is_contiguous(), "qweight is not contiguous");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(qweight.device());
  Tensor output = inplace ? qweight : at::empty_like(qweight);
  if (qweight.numel() == 0) return output;
  if (!qzeros_or_none.has_value()) {
    TORCH_CHECK(qweight.numel() * 8 % 256 == 0, "qweight.numel() * 8 % 256 != 0");
    raise_if_failed(sonar_marlin_int4_fp8_preprocess(static_cast<const uint32_t*>(qweight.const_data_ptr()), nullptr,
                                                     static_cast<uint32_t*>(output.mutable_data_ptr()),
                                                     qweight.numel(), 1, 0, current_stream(qweight)));
  } else {
    const Tensor& qzeros = qzeros_or_none.value();
    TORCH_CHECK(qweight.dim() == 2 && qzeros.dim() == 2, "qweight and qzeros must be 2-D");
    TORCH_CHECK(qweight.size(0) % 32 == 0, "size_k % 32 != 0");
    TORCH_CHECK(qzeros.is_cuda(), "qzeros is not on GPU");
    TORCH_CHECK(qzeros.scalar_type() == at::kInt, "qweight.dtype != torch.int32");
    TORCH_CHECK(qzeros.device() == qweight.device(), "qzeros is not on the same device with qweight");
    TORCH_CHECK(qzeros.is_contiguous(), "qzeros is not contiguous");
    TORCH_CHECK(qweight.size(1) == qzeros.size(1), "qweight.size(1) != qzeros.size(1)");
    TORCH_CHECK(qzeros.size(0) > 0 && qweight.size(0) % qzeros.size(0) == 0,
                "qweight.size(0) % qzeros.size(0) != 0");
    const int64_t group_size = qweight.size(0) / qzeros.size(0);
    TORCH_CHECK(group_size % 8 == 0, "group_size % 8 != 0");
    raise_if_failed(sonar_marlin_int4_fp8_preprocess(static_cast<const uint32_t*>(qweight.const_data_ptr()),
                                                     static_cast<const uint32_t*>(qzeros.const_data_ptr()),
                                                     static_cast<uint32_t*>(output.mutable_data_ptr()),
                                                     qweight.size(0), qweight.size(1), group_size,
                                                     current_stream(qweight)));
  }
  forget_memory_of(output);
  return output;
}

// ---------------------------------------------------------------- dense GEMM
void check_b_type(int64_t b_type_id) {
  TORCH_CHECK_NOT_IMPLEMENTED(
      b_type_id == SONAR_TYPE_UINT4B8 || b_type_id == SONAR_TYPE_UINT4 || b_type_id == SONAR_TYPE_UINT8B128 ||
          b_type_id == SONAR_TYPE_FLOAT8_E4M3FN || b_type_id == SONAR_TYPE_FLOAT4_E2M1F,
      "b_type_id = ", b_type_id,
      " is not built here: only uint4b8, uint8b128 (GPTQ), uint4 (AWQ), float8_e4m3fn and float4_e2m1f (MXFP4) "
      "weights are supported");
}

// 8-bit activations (marlin.cu:567-598,666-679,878-882): int8 or float8_e4m3fn `a` with one fp32
// scale per row; c takes the type of b_scales.
Tensor marlin_gemm_a8(const Tensor& a, const OptTensor& c_or_none, const Tensor& b_q_weight,
                      const OptTensor& b_bias_or_none, const Tensor& b_scales, const OptTensor& a_scales,
                      const OptTensor& global_scale, const OptTensor& b_zeros_or_none,
                      const OptTensor& g_idx_or_none, int64_t b_type_id, int64_t size_m, int64_t size_n,
                      int64_t size_k, bool is_zp_float) {
  const int a_dtype = a.scalar_type() == at::kChar ? SONAR_ADTYPE_INT8 : SONAR_ADTYPE_FP8;
  check_b_type(b_type_id);
  // MXFP4 weights with fp8 activations ("W4A8-FP4", marlin.cu:576-590): exponent-byte scales per 32
  // rows, the output type is that of c, which must be passed
  const bool f4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F;
  if (f4) {
    TORCH_CHECK(a_dtype == SONAR_ADTYPE_FP8, "MXFP4 weight + INT8 activation is not supported.");
    TORCH_CHECK(is_mx_scale_type(b_scales), "float4_e2m1f weights with 8-bit activations take float8_e8m0fnu "
                "scales (MXFP4); NVFP4 weight + INT8/FP8 activation is not supported.");
    TORCH_CHECK(c_or_none.has_value(), "c must be passed for W4A8-FP4");
    TORCH_CHECK(c_or_none->scalar_type() == at::kHalf || c_or_none->scalar_type() == at::kBFloat16,
                "unsupported c dtype");
  } else if (a_dtype == SONAR_ADTYPE_INT8) {   // marlin_utils.py:672-676
    TORCH_CHECK(b_type_id == SONAR_TYPE_UINT4B8 || b_type_id == SONAR_TYPE_UINT4,
                "W8A8-INT8 is not supported by marlin kernel.");
  } else {
    TORCH_CHECK(b_type_id == SONAR_TYPE_UINT4B8 || b_type_id == SONAR_TYPE_UINT4,
                "INT8 weight + FP8 activation is not supported.");
  }
  const at::ScalarType c_type = f4 ? c_or_none->scalar_type() : b_scales.scalar_type();
  TORCH_CHECK(c_type == at::kHalf || c_type == at::kBFloat16,
              "b_scales must be float16 or bfloat16 with 8-bit activations (their type is the type of c)");
  const int dtype = c_type == at::kHalf ? SONAR_DTYPE_F16 : SONAR_DTYPE_BF16;
  TORCH_CHECK(a_scales.has_value() && a_scales->numel() > 0,
              "the a_scales parameter must be passed for 8bit activation.");
  TORCH_CHECK(a_scales->is_cuda() && a_scales->scalar_type() == at::kFloat, "scalar type of a_scales must be float");
  TORCH_CHECK(a_scales->is_contiguous() && a_scales->numel() == size_m, "a_scales must hold one scale per row of a; "
              "got ", a_scales->numel(), " for size_m = ", size_m);
  TORCH_CHECK(!(global_scale.has_value() && global_scale->numel() > 0),
              "global_scale can only be used for nvfp4 format.");
  TORCH_CHECK_NOT_IMPLEMENTED(!is_zp_float, "is_zp_float = True is not built");
  TORCH_CHECK(!(g_idx_or_none.has_value() && g_idx_or_none->numel() > 0),
              "act-order is not supported with 8-bit activations (the reference builds no such kernel)");

  TORCH_CHECK(a.dim() == 2, "a must be 2-D");
  TORCH_CHECK(a.size(0) == size_m, "Shape mismatch: a.size(0) = ", a.size(0), ", size_m = ", size_m);
  TORCH_CHECK(a.size(1) == size_k, "Shape mismatch: a.size(1) = ", a.size(1), ", size_k = ", size_k);
  TORCH_CHECK(size_k % 16 == 0, "size_k = ", size_k, " is not divisible by tile_size = ", 16);
  TORCH_CHECK(b_q_weight.dim() == 2 && size_k / 16 == b_q_weight.size(0),
              "Shape mismatch: b_q_weight.size(0) = ", b_q_weight.size(0), ", size_k = ", size_k,
              ", tile_size = ", 16);
  TORCH_CHECK(b_q_weight.size(1) % 16 == 0, "b_q_weight.size(1) = ", b_q_weight.size(1),
              " is not divisible by tile_size = ", 16);
  const int64_t actual_size_n = b_q_weight.size(1) / 16 * 8;
  TORCH_CHECK(size_n == actual_size_n, "size_n = ", size_n, ", actual_size_n = ", actual_size_n);
  TORCH_CHECK(a.is_cuda(), "A is not on GPU");
  TORCH_CHECK(size_m == 0 || a.stride(1) == 1, "A.stride(1) is not 1");
  TORCH_CHECK(size_m == 0 || a.stride(0) % 8 == 0, "A.stride(0) must divisible by 8");
  TORCH_CHECK(((uint64_t)a.const_data_ptr()) % 16 == 0, "A must aligned to 16 bytes");
  TORCH_CHECK(b_q_weight.is_cuda(), "b_q_weight is not on GPU");
  TORCH_CHECK(b_q_weight.is_contiguous(), "b_q_weight is not contiguous");
  TORCH_CHECK(b_q_weight.scalar_type() == at::kInt, "b_q_weight type is not kInt");
  TORCH_CHECK(b_scales.is_cuda(), "b_scales is not on GPU");
  TORCH_CHECK(b_scales.is_contiguous(), "b_scales is not contiguous");

  c10::hip::HIPGuardMasqueradingAsCUDA guard(a.device());
  Tensor c;
  if (c_or_none.has_value()) {
    c = c_or_none.value();
    TORCH_CHECK(c.is_cuda(), "c is not on GPU");
    TORCH_CHECK(c.is_contiguous(), "c is not contiguous");
    TORCH_CHECK(c.size(0) == size_m, "Shape mismatch: c.size(0) = ", c.size(0), ", size_m = ", size_m);
    TORCH_CHECK(c.size(1) == size_n, "Shape mismatch: c.size(1) = ", c.size(1), ", size_n = ", size_n);
    TORCH_CHECK(c.scalar_type() == c_type, "c must have the type of b_scales with 8-bit activations");
  } else {
    c = at::empty({size_m, size_n}, b_scales.options());
  }
  if (size_m == 0) return c;

  TORCH_CHECK(b_scales.dim() == 2, "b_scales rank = ", b_scales.dim(), " is not 2");
  TORCH_CHECK(b_scales.size(1) == size_n, "b_scales dim 1 = ", b_scales.size(1), " is not size_n = ", size_n);
  const int64_t num_groups = b_scales.size(0);
  if (b_bias_or_none.has_value()) {
    const Tensor& b = b_bias_or_none.value();
    TORCH_CHECK(b.is_cuda(), "b_bias is not on GPU");
    TORCH_CHECK(b.is_contiguous(), "b_bias is not contiguous");
    TORCH_CHECK(b.size(0) == size_n, "b_bias.size(0) != size_n");
    TORCH_CHECK(b.scalar_type() == c.scalar_type(), "b_bias must have the dtype of c");
  }
  const bool has_zp = b_zeros_or_none.has_value() && b_zeros_or_none->size(-1) > 0;
  if (has_zp) {
    const Tensor& z = b_zeros_or_none.value();
    TORCH_CHECK(z.is_cuda(), "b_zeros is not on GPU");
    TORCH_CHECK(z.is_contiguous(), "b_zeros is not contiguous");
    TORCH_CHECK(b_type_id == SONAR_TYPE_UINT4, "b_type must be u4 or u8 when has_zp = True. Got = uint4b8");
    TORCH_CHECK(z.dim() == 2, "b_zeros rank = ", z.dim(), " is not 2");
    TORCH_CHECK(z.size(0) == num_groups, "b_zeros dim 0 = ", z.size(0), " is not num_groups = ", num_groups);
    TORCH_CHECK(z.size(1) == size_n / 8, "b_zeros dim 1 = ", z.size(1), " is not size_n / pack_factor = ", size_n / 8);
    TORCH_CHECK(z.scalar_type() == at::kInt, "b_zeros must be int32");
  } else {
    TORCH_CHECK(b_type_id != SONAR_TYPE_UINT4,
                "b_type must be uint4b8, uint8b128, int4, int8, float8_e4m3fn or float4_e2m1f when "
                "has_zp = False. Got = uint4");
  }
  TORCH_CHECK(size_n % 64 == 0, "size_n = ", size_n, ", is not divisible by min_thread_n = ", 64);
  TORCH_CHECK(size_k % 32 == 0, "size_k = ", size_k, " is not divisible by 32 (the k tile of 8-bit activations)");

  Tensor native = native_weights(b_q_weight, size_k, size_n, 1, 4, /*a8=*/true);
  const size_t scratch_bytes = sonar_marlin_gemm_a8_scratch_bytes(size_m, size_n, size_k, num_groups);
  Tensor scratch = at::empty({(int64_t)std::max<size_t>(scratch_bytes, 16)}, a.options().dtype(at::kByte));
  raise_if_failed(sonar_marlin_gemm_a8(
      a.const_data_ptr(), a.stride(0), a_dtype, c.mutable_data_ptr(),
      static_cast<const uint32_t*>(native.const_data_ptr()), SONAR_LAYOUT_GFX950, opt_ptr(b_bias_or_none),
      b_scales.const_data_ptr(), static_cast<const float*>(a_scales->const_data_ptr()),
      has_zp ? static_cast<const uint32_t*>(b_zeros_or_none->const_data_ptr()) : nullptr, scratch.mutable_data_ptr(),
      scratch_bytes, dtype, b_type_id, size_m, size_n, size_k, num_groups, current_stream(a)));
  return c;
}

Tensor marlin_gemm(const Tensor& a, const OptTensor& c_or_none, const Tensor& b_q_weight,
                   const OptTensor& b_bias_or_none, const Tensor& b_scales, const OptTensor& a_scales,
                   const OptTensor& global_scale, const OptTensor& b_zeros_or_none,
                   const OptTensor& g_idx_or_none, const OptTensor& perm_or_none,
                   const Tensor& workspace, int64_t b_type_id, int64_t size_m, int64_t size_n,
                   int64_t size_k, bool is_k_full, bool use_atomic_add, bool use_fp32_reduce,
                   bool is_zp_float) {
  if (a.scalar_type() == at::kChar || a.scalar_type() == at::kFloat8_e4m3fn)
    return marlin_gemm_a8(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, a_scales, global_scale,
                          b_zeros_or_none, g_idx_or_none, b_type_id, size_m, size_n, size_k, is_zp_float);
  TORCH_CHECK(a.scalar_type() == at::kHalf || a.scalar_type() == at::kBFloat16, "unsupported `a` scalar_type");
  const int dtype = dtype_code(a);
  check_b_type(b_type_id);
  TORCH_CHECK(!(a_scales.has_value() && a_scales->numel() > 0), "a_scales can only be used for 8bit activation.");
  TORCH_CHECK_NOT_IMPLEMENTED(!is_zp_float, "is_zp_float = True is not built");
  // marlin.cu:784-796
  const bool nvfp4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F && b_scales.scalar_type() == at::kFloat8_e4m3fn;
  if (global_scale.has_value() && global_scale->numel() > 0) {
    TORCH_CHECK(nvfp4, "global_scale can only be used for nvfp4 format.");
    TORCH_CHECK(global_scale->is_cuda() && global_scale->scalar_type() == at::kFloat,
                "scalar type of global_scale must be float");
  } else {
    TORCH_CHECK(!nvfp4, "the global_scale parameter must be passed for nvfp4 format.");
  }

  TORCH_CHECK(a.dim() == 2, "a must be 2-D");
  TORCH_CHECK(a.size(0) == size_m, "Shape mismatch: a.size(0) = ", a.size(0), ", size_m = ", size_m);
  TORCH_CHECK(a.size(1) == size_k, "Shape mismatch: a.size(1) = ", a.size(1), ", size_k = ", size_k);
  TORCH_CHECK(size_k % 16 == 0, "size_k = ", size_k, " is not divisible by tile_size = ", 16);
  TORCH_CHECK(b_q_weight.dim() == 2 && size_k / 16 == b_q_weight.size(0),
              "Shape mismatch: b_q_weight.size(0) = ", b_q_weight.size(0), ", size_k = ", size_k,
              ", tile_size = ", 16);
  TORCH_CHECK(b_q_weight.size(1) % 16 == 0, "b_q_weight.size(1) = ", b_q_weight.size(1),
              " is not divisible by tile_size = ", 16);
  const int bits = (b_type_id == SONAR_TYPE_UINT8B128 || b_type_id == SONAR_TYPE_FLOAT8_E4M3FN) ? 8 : 4;
  const int64_t actual_size_n = b_q_weight.size(1) / 16 * (32 / bits);
  TORCH_CHECK(size_n == actual_size_n, "size_n = ", size_n, ", actual_size_n = ", actual_size_n);

  TORCH_CHECK(a.is_cuda(), "A is not on GPU");
  TORCH_CHECK(size_m == 0 || a.stride(1) == 1, "A.stride(1) is not 1");
  TORCH_CHECK(size_m == 0 || a.stride(0) % 8 == 0, "A.stride(0) must divisible by 8");
  TORCH_CHECK(((uint64_t)a.const_data_ptr()) % 16 == 0, "A must aligned to 16 bytes");
  TORCH_CHECK(b_q_weight.is_cuda(), "b_q_weight is not on GPU");
  TORCH_CHECK(b_q_weight.is_contiguous(), "b_q_weight is not contiguous");
  TORCH_CHECK(b_q_weight.scalar_type() == at::kInt, "b_q_weight type is not kInt");
  TORCH_CHECK(b_scales.is_cuda(), "b_scales is not on GPU");
  TORCH_CHECK(b_scales.is_contiguous(), "b_scales is not contiguous");
  const bool fp4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F;
  // marlin.cu:612-617: fp8 weights with exponent-byte scales per 32 rows (MXFP8, bfloat16 activations)
  const bool mxfp8 = b_type_id == SONAR_TYPE_FLOAT8_E4M3FN && b_scales.scalar_type() == at::kFloat8_e8m0fnu;
  if (mxfp8) {
    TORCH_CHECK(a.scalar_type() == at::kBFloat16, "float8_e4m3fn weights with float8_e8m0fnu scales (MXFP8) "
                "need bfloat16 activations");
  } else if (nvfp4) {   // marlin.cu:600-611
    TORCH_CHECK(g_idx_or_none.has_value() ? g_idx_or_none->numel() == 0 : true,
                "act-order is not supported with float4_e2m1f weights");
  } else if (fp4) {
    TORCH_CHECK(is_mx_scale_type(b_scales),
                "When b_type = float4_e2m1f, b_scale scalar type must be",
                "float8_e4m3fn (for NVFP4) or float8_e8m0fnu (for MXFP4).");
  } else {
    TORCH_CHECK(b_scales.scalar_type() == a.scalar_type(),
                "scalar type of b_scales must be the same as a for 16 bit activation");
  }

  c10::hip::HIPGuardMasqueradingAsCUDA guard(a.device());
  Tensor c;
  if (c_or_none.has_value()) {
    c = c_or_none.value();
    TORCH_CHECK(c.is_cuda(), "c is not on GPU");
    TORCH_CHECK(c.is_contiguous(), "c is not contiguous");
    TORCH_CHECK(c.size(0) == size_m, "Shape mismatch: c.size(0) = ", c.size(0), ", size_m = ", size_m);
    TORCH_CHECK(c.size(1) == size_n, "Shape mismatch: c.size(1) = ", c.size(1), ", size_n = ", size_n);
    TORCH_CHECK(c.scalar_type() == a.scalar_type(),
                "scalar type of a must be the same with c for 16 bit activation");
  } else {
    c = at::empty({size_m, size_n}, a.options());
  }
  if (size_m == 0) return c;

  TORCH_CHECK(b_scales.dim() == 2, "b_scales rank = ", b_scales.dim(), " is not 2");
  TORCH_CHECK(b_scales.size(1) == size_n, "b_scales dim 1 = ", b_scales.size(1), " is not size_n = ", size_n);
  const int64_t num_groups = b_scales.size(0);

  const int32_t* g_idx = nullptr;
  const int32_t* perm = nullptr;
  if (g_idx_or_none.has_value() && perm_or_none.has_value()) {
    const Tensor& g = g_idx_or_none.value();
    const Tensor& p = perm_or_none.value();
    TORCH_CHECK(g.is_cuda(), "g_idx is not on GPU");
    TORCH_CHECK(g.is_contiguous(), "g_idx is not contiguous");
    TORCH_CHECK(p.is_cuda(), "perm is not on GPU");
    TORCH_CHECK(p.is_contiguous(), "perm is not contiguous");
    TORCH_CHECK((g.size(-1) == 0 && p.size(-1) == 0) || (g.size(-1) == size_k && p.size(-1) == size_k),
                "Unexpected g_idx.size(-1) = ", g.size(-1), " and perm.size(-1) = ", p.size(-1),
                ", where size_k = ", size_k);
    if (g.size(-1) > 0) {
      TORCH_CHECK(g.scalar_type() == at::kInt && p.scalar_type() == at::kInt, "g_idx and perm must be int32");
      g_idx = static_cast<const int32_t*>(g.const_data_ptr());
      perm = static_cast<const int32_t*>(p.const_data_ptr());
    }
  }

  if (b_bias_or_none.has_value()) {
    const Tensor& b = b_bias_or_none.value();
    TORCH_CHECK(b.is_cuda(), "b_bias is not on GPU");
    TORCH_CHECK(b.is_contiguous(), "b_bias is not contiguous");
    TORCH_CHECK(b.size(0) == size_n, "b_bias.size(0) != size_n");
    TORCH_CHECK(b.stride(0) == 1, "b_bias.stride(0) != 1");
    TORCH_CHECK(b.scalar_type() == a.scalar_type(), "b_bias must have the dtype of a");
  }

  const bool has_zp = b_zeros_or_none.has_value() && b_zeros_or_none->size(-1) > 0;
  if (has_zp) {
    const Tensor& z = b_zeros_or_none.value();
    TORCH_CHECK(z.is_cuda(), "b_zeros is not on GPU");
    TORCH_CHECK(z.is_contiguous(), "b_zeros is not contiguous");
    TORCH_CHECK(b_type_id == SONAR_TYPE_UINT4, "b_type must be u4 or u8 when has_zp = True. Got = uint4b8");
    TORCH_CHECK(z.dim() == 2, "b_zeros rank = ", z.dim(), " is not 2");
    TORCH_CHECK(z.size(0) == num_groups, "b_zeros dim 0 = ", z.size(0), " is not num_groups = ", num_groups);
    TORCH_CHECK(z.size(1) == size_n / 8, "b_zeros dim 1 = ", z.size(1),
                " is not size_n / pack_factor = ", size_n / 8);
    TORCH_CHECK(z.scalar_type() == at::kInt, "b_zeros must be int32");
  } else {
    TORCH_CHECK(b_type_id != SONAR_TYPE_UINT4,
                "b_type must be uint4b8, uint8b128, int4, int8, float8_e4m3fn or float4_e2m1f when "
                "has_zp = False. Got = uint4");
  }

  TORCH_CHECK(size_n % 64 == 0, "size_n = ", size_n, ", is not divisible by min_thread_n = ", 64);
  TORCH_CHECK(workspace.is_cuda() && workspace.scalar_type() == at::kInt && workspace.is_contiguous(),
              "workspace must be a contiguous int32 GPU tensor");

  Tensor native = native_weights(b_q_weight, size_k, size_n, 1, bits);
  size_t scratch_bytes = sonar_marlin_gemm_scratch_bytes(size_m, size_n, size_k);
  if (perm != nullptr) scratch_bytes += (size_t)size_m * size_k * 2;  // room for the column-permuted copy of A
  Tensor scratch = at::empty({(int64_t)scratch_bytes}, a.options().dtype(at::kByte));

  if (nvfp4) {
    TORCH_CHECK(size_k == 16 * num_groups, "float4_e2m1f weights with float8_e4m3fn scales (NVFP4) take one scale "
                "per group of 16 rows; got size_k = ", size_k, ", b_scales.size(0) = ", num_groups);
    raise_if_failed(sonar_marlin_gemm_nvfp4(
        a.const_data_ptr(), a.stride(0), c.mutable_data_ptr(),
        static_cast<const uint32_t*>(native.const_data_ptr()), SONAR_LAYOUT_GFX950, opt_ptr(b_bias_or_none),
        nvfp4_scales_as_16bit(b_scales, a.scalar_type()).const_data_ptr(),
        static_cast<const float*>(global_scale->const_data_ptr()),
        static_cast<int32_t*>(workspace.mutable_data_ptr()), workspace.numel(), scratch.mutable_data_ptr(),
        scratch_bytes, dtype, size_m, size_n, size_k, num_groups, current_stream(a)));
    return c;
  }
  raise_if_failed(sonar_marlin_gemm(
      a.const_data_ptr(), a.stride(0), c.mutable_data_ptr(),
      static_cast<const uint32_t*>(native.const_data_ptr()), SONAR_LAYOUT_GFX950,
      opt_ptr(b_bias_or_none),
      (fp4 || mxfp8 ? mx_scales_as_bf16(b_scales, mxfp8 ? 120 : 0) : b_scales).const_data_ptr(),
      has_zp ? static_cast<const uint32_t*>(b_zeros_or_none->const_data_ptr()) : nullptr, g_idx, perm,
      static_cast<int32_t*>(workspace.mutable_data_ptr()), workspace.numel(), scratch.mutable_data_ptr(),
      scratch_bytes, dtype, b_type_id, size_m, size_n, size_k, num_groups, is_k_full ? 1 : 0,
      use_atomic_add ? 1 : 0, use_fp32_reduce ? 1 : 0, current_stream(a)));
  return c;
}

// ---------------------------------------------------------------- grouped GEMM
// 8-bit activations (moe/marlin_moe_wna16/ops.cu: the same type resolution as marlin.cu:567-598).
Tensor moe_wna16_marlin_gemm_a8(const Tensor& a, const OptTensor& c_or_none, const Tensor& b_q_weight,
                                const OptTensor& b_bias_or_none, const Tensor& b_scales, const OptTensor& a_scales,
                                const OptTensor& global_scale, const OptTensor& b_zeros_or_none,
                                const OptTensor& g_idx_or_none, const Tensor& sorted_token_ids,
                                const Tensor& expert_ids, const Tensor& num_tokens_past_padded,
                                const Tensor& topk_weights, int64_t moe_block_size, int64_t top_k,
                                bool mul_topk_weights, int64_t b_type_id, int64_t size_m, int64_t size_n,
                                int64_t size_k, bool is_zp_float) {
  const int a_dtype = a.scalar_type() == at::kChar ? SONAR_ADTYPE_INT8 : SONAR_ADTYPE_FP8;
  check_b_type(b_type_id);
  const bool f4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F;   // MXFP4 experts with fp8 tokens: c gives the output type
  if (f4) {
    TORCH_CHECK(a_dtype == SONAR_ADTYPE_FP8, "MXFP4 weight + INT8 activation is not supported.");
    TORCH_CHECK(is_mx_scale_type(b_scales), "float4_e2m1f weights with 8-bit activations take float8_e8m0fnu "
                "scales (MXFP4); NVFP4 weight + INT8/FP8 activation is not supported.");
    TORCH_CHECK(c_or_none.has_value(), "c must be passed for W4A8-FP4");
  } else {
    TORCH_CHECK(b_type_id == SONAR_TYPE_UINT4B8 || b_type_id == SONAR_TYPE_UINT4,
                a_dtype == SONAR_ADTYPE_INT8 ? "W8A8-INT8 is not supported by marlin kernel."
                                             : "INT8 weight + FP8 activation is not supported.");
  }
  const at::ScalarType c_type = f4 ? c_or_none->scalar_type() : b_scales.scalar_type();
  TORCH_CHECK(c_type == at::kHalf || c_type == at::kBFloat16,
              "b_scales must be float16 or bfloat16 with 8-bit activations (their type is the type of c)");
  const int dtype = c_type == at::kHalf ? SONAR_DTYPE_F16 : SONAR_DTYPE_BF16;
  TORCH_CHECK(a_scales.has_value() && a_scales->numel() > 0,
              "the a_scales parameter must be passed for 8bit activation.");
  TORCH_CHECK(a_scales->is_cuda() && a_scales->scalar_type() == at::kFloat && a_scales->is_contiguous(),
              "scalar type of a_scales must be float");
  TORCH_CHECK(a_scales->numel() == size_m, "a_scales must hold one scale per row of a; got ", a_scales->numel(),
              " for size_m = ", size_m);
  TORCH_CHECK(!(global_scale.has_value() && global_scale->numel() > 0),
              "global_scale can only be used for nvfp4 format.");
  TORCH_CHECK_NOT_IMPLEMENTED(!is_zp_float, "is_zp_float = True is not built");
  TORCH_CHECK(!(g_idx_or_none.has_value() && g_idx_or_none->numel() > 0),
              "act-order is not supported with 8-bit activations (the reference builds no such kernel)");
  TORCH_CHECK(moe_block_size == 8 || moe_block_size % 16 == 0, "unsupported moe_block_size=", moe_block_size);
  TORCH_CHECK(moe_block_size >= 8 && moe_block_size <= 64, "unsupported moe_block_size=", moe_block_size);
  TORCH_CHECK(a.dim() == 2 && a.size(0) == size_m, "Shape mismatch: a.size(0) = ", a.size(0),
              ", size_m = ", size_m);
  TORCH_CHECK(a.size(1) == size_k, "Shape mismatch: a.size(1) = ", a.size(1), ", size_k = ", size_k);
  TORCH_CHECK(a.is_cuda() && a.is_contiguous(), "A is not a contiguous GPU tensor");
  TORCH_CHECK(b_q_weight.dim() == 3, "b_q_weight must be (E, K/16, 2N)");
  const int64_t experts = b_q_weight.size(0);
  TORCH_CHECK(size_k % 32 == 0 && size_k / 16 == b_q_weight.size(1),
              "Shape mismatch: b_q_weight.size(1) = ", b_q_weight.size(1), ", size_k = ", size_k,
              ", tile_size = ", 16);
  TORCH_CHECK(b_q_weight.size(2) % 16 == 0 && b_q_weight.size(2) / 16 * 8 == size_n,
              "size_n = ", size_n, ", actual_size_n = ", b_q_weight.size(2) / 16 * 8);
  TORCH_CHECK(b_q_weight.is_cuda() && b_q_weight.is_contiguous() && b_q_weight.scalar_type() == at::kInt,
              "b_q_weight must be a contiguous int32 GPU tensor");
  TORCH_CHECK(b_scales.is_cuda() && b_scales.is_contiguous(), "b_scales is not a contiguous GPU tensor");
  TORCH_CHECK(b_scales.dim() == 3 && b_scales.size(0) == experts, "b_scales rank = ", b_scales.dim(), " is not 3");
  TORCH_CHECK(b_scales.size(2) == size_n, "b_scales dim 2 = ", b_scales.size(2), " is not size_n = ", size_n);
  const int64_t num_groups = b_scales.size(1);

  c10::hip::HIPGuardMasqueradingAsCUDA guard(a.device());
  Tensor c;
  if (c_or_none.has_value()) {
    c = c_or_none.value();
    TORCH_CHECK(c.is_cuda() && c.is_contiguous(), "c is not a contiguous GPU tensor");
    TORCH_CHECK(c.size(0) == size_m * top_k, "Shape mismatch: c.size(0) = ", c.size(0),
                ", size_m * topk = ", size_m * top_k);
    TORCH_CHECK(c.size(1) == size_n, "Shape mismatch: c.size(1) = ", c.size(1), ", size_n = ", size_n);
    TORCH_CHECK(c.scalar_type() == c_type, "c must have the type of b_scales with 8-bit activations");
  } else {
    c = at::empty({size_m * top_k, size_n}, b_scales.options());
  }
  if (size_m == 0) return c;
  if (b_bias_or_none.has_value()) {
    const Tensor& b = b_bias_or_none.value();
    TORCH_CHECK(b.is_cuda() && b.is_contiguous(), "b_bias is not a contiguous GPU tensor");
    TORCH_CHECK(b.size(-1) == size_n, "b_bias.size(-1) != size_n");
    TORCH_CHECK(b.scalar_type() == c.scalar_type(), "b_bias must have the dtype of c");
  }
  const bool has_zp = b_zeros_or_none.has_value() && b_zeros_or_none->size(-1) > 0;
  if (has_zp) {
    const Tensor& z = b_zeros_or_none.value();
    TORCH_CHECK(z.is_cuda() && z.is_contiguous() && z.scalar_type() == at::kInt,
                "b_zeros must be a contiguous int32 GPU tensor");
    TORCH_CHECK(b_type_id == SONAR_TYPE_UINT4, "b_type must be u4 or u8 when has_zp = True. Got = uint4b8");
    TORCH_CHECK(z.dim() == 3 && z.size(1) == num_groups && z.size(2) == size_n / 8,
                "b_zeros must be (E, num_groups, size_n / 8)");
  } else {
    TORCH_CHECK(b_type_id != SONAR_TYPE_UINT4,
                "b_type must be uint4b8, uint8b128 or float8_e4m3fn when has_zp = False. Got = uint4");
  }
  TORCH_CHECK(sorted_token_ids.is_cuda() && sorted_token_ids.scalar_type() == at::kInt &&
                  sorted_token_ids.is_contiguous(), "sorted_token_ids must be a contiguous int32 GPU tensor");
  TORCH_CHECK(expert_ids.is_cuda() && expert_ids.scalar_type() == at::kInt && expert_ids.is_contiguous(),
              "expert_ids must be a contiguous int32 GPU tensor");
  TORCH_CHECK(num_tokens_past_padded.is_cuda() && num_tokens_past_padded.scalar_type() == at::kInt,
              "num_tokens_past_padded must be an int32 GPU tensor");
  TORCH_CHECK(topk_weights.is_cuda() && topk_weights.scalar_type() == at::kFloat &&
                  topk_weights.is_contiguous(), "topk_weights must be a contiguous float32 GPU tensor");

  Tensor native = native_weights(b_q_weight, size_k, size_n, experts, 4, /*a8=*/true);
  raise_if_failed(sonar_moe_wna16_marlin_gemm_a8(
      a.const_data_ptr(), a_dtype, c.mutable_data_ptr(), static_cast<const uint32_t*>(native.const_data_ptr()),
      SONAR_LAYOUT_GFX950, opt_ptr(b_bias_or_none), b_scales.const_data_ptr(),
      static_cast<const float*>(a_scales->const_data_ptr()),
      has_zp ? static_cast<const uint32_t*>(b_zeros_or_none->const_data_ptr()) : nullptr,
      static_cast<const int32_t*>(sorted_token_ids.const_data_ptr()), sorted_token_ids.numel(),
      static_cast<const int32_t*>(expert_ids.const_data_ptr()),
      static_cast<const int32_t*>(num_tokens_past_padded.const_data_ptr()),
      static_cast<const float*>(topk_weights.const_data_ptr()), moe_block_size, top_k, mul_topk_weights ? 1 : 0,
      experts, dtype, b_type_id, size_m, size_n, size_k, num_groups, current_stream(a)));
  return c;
}

Tensor moe_wna16_marlin_gemm(
    Tensor& a, const OptTensor& c_or_none, Tensor& b_q_weight, const OptTensor& b_bias_or_none,
    Tensor& b_scales, const OptTensor& a_scales, const OptTensor& global_scale,
    const OptTensor& b_zeros_or_none, const OptTensor& g_idx_or_none, const OptTensor& perm_or_none,
    Tensor& workspace, const Tensor& sorted_token_ids, Tensor& expert_ids,
    Tensor& num_tokens_past_padded, Tensor& topk_weights, int64_t moe_block_size, int64_t top_k,
    bool mul_topk_weights, int64_t b_type_id, int64_t size_m, int64_t size_n, int64_t size_k,
    bool is_k_full, bool use_atomic_add, bool use_fp32_reduce, bool is_zp_float, int64_t thread_k,
    int64_t thread_n, int64_t blocks_per_sm) {
  (void)thread_k;
  (void)thread_n;
  (void)blocks_per_sm;
  if (a.scalar_type() == at::kChar || a.scalar_type() == at::kFloat8_e4m3fn)
    return moe_wna16_marlin_gemm_a8(a, c_or_none, b_q_weight, b_bias_or_none, b_scales, a_scales, global_scale,
                                    b_zeros_or_none, g_idx_or_none, sorted_token_ids, expert_ids,
                                    num_tokens_past_padded, topk_weights, moe_block_size, top_k, mul_topk_weights,
                                    b_type_id, size_m, size_n, size_k, is_zp_float);
  TORCH_CHECK(a.scalar_type() == at::kHalf || a.scalar_type() == at::kBFloat16, "unsupported `a` scalar_type");
  const int dtype = dtype_code(a);
  check_b_type(b_type_id);
  TORCH_CHECK(!(a_scales.has_value() && a_scales->numel() > 0), "a_scales can only be used for 8bit activation.");
  TORCH_CHECK_NOT_IMPLEMENTED(!is_zp_float, "is_zp_float = True is not built");
  // marlin_moe_wna16/ops.cu: the global scale goes with NVFP4 and only with it
  const bool nvfp4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F && b_scales.scalar_type() == at::kFloat8_e4m3fn;
  if (global_scale.has_value() && global_scale->numel() > 0) {
    TORCH_CHECK(nvfp4, "global_scale can only be used for nvfp4 format.");
    TORCH_CHECK(global_scale->is_cuda() && global_scale->scalar_type() == at::kFloat &&
                    global_scale->is_contiguous(), "scalar type of global_scale must be float");
    TORCH_CHECK(global_scale->numel() == b_q_weight.size(0), "global_scale must hold one number per expert");
  } else {
    TORCH_CHECK(!nvfp4, "the global_scale parameter must be passed for nvfp4 format.");
  }
  TORCH_CHECK(moe_block_size == 8 || moe_block_size % 16 == 0, "unsupported moe_block_size=", moe_block_size);
  TORCH_CHECK(moe_block_size >= 8 && moe_block_size <= 64, "unsupported moe_block_size=", moe_block_size);

  TORCH_CHECK(a.dim() == 2 && a.size(0) == size_m, "Shape mismatch: a.size(0) = ", a.size(0),
              ", size_m = ", size_m);
  TORCH_CHECK(a.size(1) == size_k, "Shape mismatch: a.size(1) = ", a.size(1), ", size_k = ", size_k);
  TORCH_CHECK(a.is_cuda() && a.is_contiguous(), "A is not a contiguous GPU tensor");
  TORCH_CHECK(b_q_weight.dim() == 3, "b_q_weight must be (E, K/16, 2N)");
  const int64_t experts = b_q_weight.size(0);
  TORCH_CHECK(size_k % 16 == 0 && size_k / 16 == b_q_weight.size(1),
              "Shape mismatch: b_q_weight.size(1) = ", b_q_weight.size(1), ", size_k = ", size_k,
              ", tile_size = ", 16);
  const int bits = (b_type_id == SONAR_TYPE_UINT8B128 || b_type_id == SONAR_TYPE_FLOAT8_E4M3FN) ? 8 : 4;
  const int64_t pack_factor = 32 / bits;
  TORCH_CHECK(b_q_weight.size(2) % 16 == 0 && b_q_weight.size(2) / 16 * pack_factor == size_n,
              "size_n = ", size_n, ", actual_size_n = ", b_q_weight.size(2) / 16 * pack_factor);
  TORCH_CHECK(b_q_weight.is_cuda() && b_q_weight.is_contiguous() && b_q_weight.scalar_type() == at::kInt,
              "b_q_weight must be a contiguous int32 GPU tensor");
  TORCH_CHECK(b_scales.is_cuda() && b_scales.is_contiguous(), "b_scales is not a contiguous GPU tensor");
  TORCH_CHECK(b_scales.dim() == 3 && b_scales.size(0) == experts, "b_scales rank = ", b_scales.dim(), " is not 3");
  TORCH_CHECK(b_scales.size(2) == size_n, "b_scales dim 2 = ", b_scales.size(2), " is not size_n = ", size_n);
  const bool fp4 = b_type_id == SONAR_TYPE_FLOAT4_E2M1F;
  const bool mxfp8 = b_type_id == SONAR_TYPE_FLOAT8_E4M3FN && b_scales.scalar_type() == at::kFloat8_e8m0fnu;
  if (mxfp8) {
    TORCH_CHECK(a.scalar_type() == at::kBFloat16, "float8_e4m3fn weights with float8_e8m0fnu scales (MXFP8) "
                "need bfloat16 activations");
  } else if (nvfp4) {
    TORCH_CHECK(b_scales.size(1) * 16 == size_k, "float4_e2m1f weights with float8_e4m3fn scales (NVFP4) take one "
                "scale per group of 16 rows; got size_k = ", size_k, ", b_scales.size(1) = ", b_scales.size(1));
  } else if (fp4) {
    TORCH_CHECK(is_mx_scale_type(b_scales),
                "When b_type = float4_e2m1f, b_scale scalar type must be",
                "float8_e4m3fn (for NVFP4) or float8_e8m0fnu (for MXFP4).");
  } else {
    TORCH_CHECK(b_scales.scalar_type() == a.scalar_type(), "b_scales must have the dtype of a");
  }
  const int64_t num_groups = b_scales.size(1);

  c10::hip::HIPGuardMasqueradingAsCUDA guard(a.device());
  Tensor c;
  if (c_or_none.has_value()) {
    c = c_or_none.value();
    TORCH_CHECK(c.is_cuda() && c.is_contiguous(), "c is not a contiguous GPU tensor");
    TORCH_CHECK(c.size(0) == size_m * top_k, "Shape mismatch: c.size(0) = ", c.size(0),
                ", size_m * topk = ", size_m * top_k);
    TORCH_CHECK(c.size(1) == size_n, "Shape mismatch: c.size(1) = ", c.size(1), ", size_n = ", size_n);
    TORCH_CHECK(c.scalar_type() == a.scalar_type(), "c must have the dtype of a");
  } else {
    c = at::empty({size_m * top_k, size_n}, a.options());
  }
  if (size_m == 0) return c;

  const int32_t* g_idx = nullptr;
  const int32_t* perm = nullptr;
  if (g_idx_or_none.has_value() && perm_or_none.has_value() && g_idx_or_none->size(-1) > 0) {
    const Tensor& g = g_idx_or_none.value();
    const Tensor& p = perm_or_none.value();
    TORCH_CHECK(g.is_cuda() && g.is_contiguous() && p.is_cuda() && p.is_contiguous(),
                "g_idx and perm must be contiguous GPU tensors");
    TORCH_CHECK(g.size(-1) == size_k && p.size(-1) == size_k, "Unexpected g_idx.size(-1) = ", g.size(-1),
                " and perm.size(-1) = ", p.size(-1), ", where size_k = ", size_k);
    TORCH_CHECK(g.scalar_type() == at::kInt && p.scalar_type() == at::kInt, "g_idx and perm must be int32");
    g_idx = static_cast<const int32_t*>(g.const_data_ptr());
    perm = static_cast<const int32_t*>(p.const_data_ptr());
  }
  if (b_bias_or_none.has_value()) {
    const Tensor& b = b_bias_or_none.value();
    TORCH_CHECK(b.is_cuda() && b.is_contiguous(), "b_bias is not a contiguous GPU tensor");
    TORCH_CHECK(b.size(-1) == size_n, "b_bias.size(-1) != size_n");
    TORCH_CHECK(b.scalar_type() == a.scalar_type(), "b_bias must have the dtype of a");
  }
  const bool has_zp = b_zeros_or_none.has_value() && b_zeros_or_none->size(-1) > 0;
  if (has_zp) {
    const Tensor& z = b_zeros_or_none.value();
    TORCH_CHECK(z.is_cuda() && z.is_contiguous() && z.scalar_type() == at::kInt,
                "b_zeros must be a contiguous int32 GPU tensor");
    TORCH_CHECK(b_type_id == SONAR_TYPE_UINT4, "b_type must be u4 or u8 when has_zp = True. Got = uint4b8");
    TORCH_CHECK(z.dim() == 3 && z.size(1) == num_groups && z.size(2) == size_n / 8,
                "b_zeros must be (E, num_groups, size_n / 8)");
  } else {
    TORCH_CHECK(b_type_id != SONAR_TYPE_UINT4,
                "b_type must be uint4b8, uint8b128 or float8_e4m3fn when has_zp = False. Got = uint4");
  }
  TORCH_CHECK(sorted_token_ids.is_cuda() && sorted_token_ids.scalar_type() == at::kInt &&
                  sorted_token_ids.is_contiguous(), "sorted_token_ids must be a contiguous int32 GPU tensor");
  TORCH_CHECK(expert_ids.is_cuda() && expert_ids.scalar_type() == at::kInt && expert_ids.is_contiguous(),
              "expert_ids must be a contiguous int32 GPU tensor");
  TORCH_CHECK(num_tokens_past_padded.is_cuda() && num_tokens_past_padded.scalar_type() == at::kInt,
              "num_tokens_past_padded must be an int32 GPU tensor");
  TORCH_CHECK(topk_weights.is_cuda() && topk_weights.scalar_type() == at::kFloat &&
                  topk_weights.is_contiguous(), "topk_weights must be a contiguous float32 GPU tensor");
  TORCH_CHECK(workspace.is_cuda() && workspace.scalar_type() == at::kInt && workspace.is_contiguous(),
              "workspace must be a contiguous int32 GPU tensor");

  Tensor native = native_weights(b_q_weight, size_k, size_n, experts, bits);
  size_t scratch_bytes =
      sonar_moe_marlin_gemm_scratch_bytes(sorted_token_ids.numel(), moe_block_size, size_n, size_k);
  // act-order: room for the column-permuted copy of A, one row per slot, behind the table of row tiles
  if (perm != nullptr)
    scratch_bytes = ((scratch_bytes + 255) & ~(size_t)255) + (size_t)sorted_token_ids.numel() * size_k * 2;
  Tensor scratch;
  if (scratch_bytes > 0) scratch = at::empty({(int64_t)scratch_bytes}, a.options().dtype(at::kByte));

  if (nvfp4) {
    TORCH_CHECK(perm == nullptr, "act-order is not supported with float4_e2m1f weights");
    raise_if_failed(sonar_moe_wna16_marlin_gemm_nvfp4(
        a.const_data_ptr(), c.mutable_data_ptr(), static_cast<const uint32_t*>(native.const_data_ptr()),
        SONAR_LAYOUT_GFX950, opt_ptr(b_bias_or_none),
        nvfp4_scales_as_16bit(b_scales, a.scalar_type()).const_data_ptr(),
        static_cast<const float*>(global_scale->const_data_ptr()),
        scratch_bytes > 0 ? scratch.mutable_data_ptr() : nullptr, scratch_bytes,
        static_cast<const int32_t*>(sorted_token_ids.const_data_ptr()), sorted_token_ids.numel(),
        static_cast<const int32_t*>(expert_ids.const_data_ptr()),
        static_cast<const int32_t*>(num_tokens_past_padded.const_data_ptr()),
        static_cast<const float*>(topk_weights.const_data_ptr()), moe_block_size, top_k, mul_topk_weights ? 1 : 0,
        experts, dtype, size_m, size_n, size_k, num_groups, current_stream(a)));
    return c;
  }
  raise_if_failed(sonar_moe_wna16_marlin_gemm(
      a.const_data_ptr(), c.mutable_data_ptr(), static_cast<const uint32_t*>(native.const_data_ptr()),
      SONAR_LAYOUT_GFX950, opt_ptr(b_bias_or_none),
      (fp4 || mxfp8 ? mx_scales_as_bf16(b_scales, mxfp8 ? 120 : 0) : b_scales).const_data_ptr(),
      has_zp ? static_cast<const uint32_t*>(b_zeros_or_none->const_data_ptr()) : nullptr, g_idx, perm,
      static_cast<int32_t*>(workspace.mutable_data_ptr()), workspace.numel(),
      scratch_bytes > 0 ? scratch.mutable_data_ptr() : nullptr, scratch_bytes,
      static_cast<const int32_t*>(sorted_token_ids.const_data_ptr()),
      sorted_token_ids.numel(), static_cast<const int32_t*>(expert_ids.const_data_ptr()),
      static_cast<const int32_t*>(num_tokens_past_padded.const_data_ptr()),
      static_cast<const float*>(topk_weights.const_data_ptr()), moe_block_size, top_k,
      mul_topk_weights ? 1 : 0, experts, dtype, b_type_id, size_m, size_n, size_k, num_groups,
      is_k_full ? 1 : 0, use_atomic_add ? 1 : 0, use_fp32_reduce ? 1 : 0, current_stream(a)));
  return c;
}

// ---------------------------------------------------------------- MoE helper ops
void moe_align_block_size(const Tensor& topk_ids, int64_t num_experts, int64_t block_size,
                          Tensor& sorted_token_ids, Tensor& experts_ids, Tensor& num_tokens_post_pad,
                          const OptTensor& maybe_expert_map) {
  TORCH_CHECK(topk_ids.is_cuda() && topk_ids.is_contiguous() && topk_ids.scalar_type() == at::kInt,
              "topk_ids must be a contiguous int32 GPU tensor");
  for (const Tensor* t : {&sorted_token_ids, &experts_ids, &num_tokens_post_pad})
    TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->scalar_type() == at::kInt,
                "outputs must be contiguous int32 GPU tensors");
  const int32_t* map = nullptr;
  if (maybe_expert_map.has_value()) {
    const Tensor& m = maybe_expert_map.value();
    TORCH_CHECK(m.is_cuda() && m.is_contiguous() && m.scalar_type() == at::kInt && m.numel() == num_experts,
                "expert_map must be a contiguous int32 GPU tensor of num_experts entries");
    map = static_cast<const int32_t*>(m.const_data_ptr());
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(topk_ids.device());
  Tensor offsets = at::empty({num_experts}, topk_ids.options());
  raise_if_failed(sonar_moe_align_block_size(
      static_cast<const int32_t*>(topk_ids.const_data_ptr()), topk_ids.numel(), num_experts, block_size,
      static_cast<int32_t*>(sorted_token_ids.mutable_data_ptr()), sorted_token_ids.numel(),
      static_cast<int32_t*>(experts_ids.mutable_data_ptr()), experts_ids.numel(),
      static_cast<int32_t*>(num_tokens_post_pad.mutable_data_ptr()), map,
      static_cast<int32_t*>(offsets.mutable_data_ptr()), current_stream(topk_ids)));
}

void silu_and_mul(Tensor& result, const Tensor& input) {
  TORCH_CHECK(input.is_cuda() && input.is_contiguous() && result.is_cuda() && result.is_contiguous(),
              "silu_and_mul needs contiguous GPU tensors");
  TORCH_CHECK(result.scalar_type() == input.scalar_type(), "result must have the dtype of input");
  const int64_t d = input.size(-1) / 2;
  TORCH_CHECK(input.size(-1) == 2 * d && result.size(-1) == d && result.numel() * 2 == input.numel(),
              "result must be input with the last dimension halved");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
  raise_if_failed(sonar_silu_and_mul(result.mutable_data_ptr(), input.const_data_ptr(), input.numel() / (2 * d),
                                     d, dtype_code(input), current_stream(input)));
}

// The reference's other gated activations (fused_moe/activation.py:128-205), schemas as in
// csrc/libtorch_stable/torch_bindings.cpp:640-680 of the reference.
void gated_activation(Tensor& result, const Tensor& input, int kind, double limit, double alpha, double beta,
                      const char* name) {
  TORCH_CHECK(input.is_cuda() && input.is_contiguous() && result.is_cuda() && result.is_contiguous(), name,
              " needs contiguous GPU tensors");
  TORCH_CHECK(result.scalar_type() == input.scalar_type(), "result must have the dtype of input");
  const int64_t d = input.size(-1) / 2;
  TORCH_CHECK(input.size(-1) == 2 * d && result.size(-1) == d && result.numel() * 2 == input.numel(),
              "result must be input with the last dimension halved");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
  raise_if_failed(sonar_moe_activation(result.mutable_data_ptr(), input.const_data_ptr(), input.numel() / (2 * d), d,
                                       kind, (float)limit, (float)alpha, (float)beta, dtype_code(input),
                                       current_stream(input)));
}
void silu_and_mul_with_clamp(Tensor& result, const Tensor& input, double limit, double alpha, double beta) {
  gated_activation(result, input, SONAR_ACT_SILU_CLAMP, limit, alpha, beta, "silu_and_mul_with_clamp");
}
void gelu_and_mul(Tensor& out, const Tensor& input) { gated_activation(out, input, SONAR_ACT_GELU, 0, 1, 0, "gelu_and_mul"); }
void gelu_tanh_and_mul(Tensor& out, const Tensor& input) {
  gated_activation(out, input, SONAR_ACT_GELU_TANH, 0, 1, 0, "gelu_tanh_and_mul");
}
void swigluoai_and_mul(Tensor& out, const Tensor& input, double alpha, double limit) {
  gated_activation(out, input, SONAR_ACT_SWIGLUOAI, limit, alpha, 0, "swigluoai_and_mul");
}
void situ_and_mul(Tensor& out, const Tensor& input, double beta, double linear_beta) {
  gated_activation(out, input, SONAR_ACT_SITU, 0, beta, linear_beta, "situ_and_mul");
}
void swiglustep_and_mul(Tensor& out, const Tensor& input, double limit) {
  gated_activation(out, input, SONAR_ACT_SWIGLUSTEP, limit, 1, 0, "swiglustep_and_mul");
}

void moe_sum(const Tensor& input, Tensor& output) {
  TORCH_CHECK(input.is_cuda() && input.is_contiguous() && output.is_cuda() && output.is_contiguous(),
              "moe_sum needs contiguous GPU tensors");
  TORCH_CHECK(input.dim() == 3 && output.dim() == 2 && output.size(0) == input.size(0) &&
                  output.size(1) == input.size(2), "moe_sum: input [tokens, topk, d], output [tokens, d]");
  TORCH_CHECK(output.scalar_type() == input.scalar_type(), "output must have the dtype of input");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(input.device());
  raise_if_failed(sonar_moe_sum(output.mutable_data_ptr(), input.const_data_ptr(), input.size(0), input.size(1),
                                input.size(2), dtype_code(input), current_stream(input)));
}

// Per-token quantisation of the activations of the W4A8 GEMM: (codes of x's shape, float32
// scales (..., 1)).
std::tuple<Tensor, Tensor> per_token_quant(const Tensor& x, bool fp8) {
  TORCH_CHECK(x.is_cuda(), "x is not on GPU");
  TORCH_CHECK(x.dim() >= 1 && x.size(-1) > 0, "x must have a non-empty last dimension");
  int dtype;
  if (x.scalar_type() == at::kHalf) dtype = SONAR_DTYPE_F16;
  else if (x.scalar_type() == at::kBFloat16) dtype = SONAR_DTYPE_BF16;
  else if (x.scalar_type() == at::kFloat) dtype = SONAR_DTYPE_F32;
  else TORCH_CHECK(false, "per-token quantisation takes float16, bfloat16 or float32; got ", x.scalar_type());
  const int64_t cols = x.size(-1);
  const Tensor x2 = x.reshape({-1, cols});
  const Tensor src = x2.stride(1) == 1 ? x2 : x2.contiguous();
  const int64_t rows = src.size(0);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  Tensor q = at::empty(x.sizes(), x.options().dtype(fp8 ? at::kFloat8_e4m3fn : at::kChar));
  auto scale_shape = x.sizes().vec();
  scale_shape.back() = 1;
  Tensor scales = at::empty(scale_shape, x.options().dtype(at::kFloat));
  if (fp8)
    raise_if_failed(sonar_per_token_quant_fp8(src.const_data_ptr(), dtype, rows ? src.stride(0) : cols,
                                              static_cast<uint8_t*>(q.mutable_data_ptr()),
                                              static_cast<float*>(scales.mutable_data_ptr()), rows, cols,
                                              current_stream(x)));
  else
    raise_if_failed(sonar_per_token_quant_int8(src.const_data_ptr(), dtype, rows ? src.stride(0) : cols,
                                               static_cast<int8_t*>(q.mutable_data_ptr()),
                                               static_cast<float*>(scales.mutable_data_ptr()), rows, cols,
                                               current_stream(x)));
  return {q, scales};
}
std::tuple<Tensor, Tensor> per_token_quant_int8(const Tensor& x) { return per_token_quant(x, false); }
std::tuple<Tensor, Tensor> per_token_quant_fp8(const Tensor& x) { return per_token_quant(x, true); }

}  // namespace

// Ops every build of the reference already has under _C / _moe_C (they are not
// CUDA-only there); registered under a namespace of their own so that loading
// this library next to the reference's extension defines nothing twice.
TORCH_LIBRARY(sonar_amd, m) {
  m.def(
      "moe_align_block_size(Tensor topk_ids, int num_experts, int block_size, Tensor! sorted_token_ids, "
      "Tensor! experts_ids, Tensor! num_tokens_post_pad, Tensor? maybe_expert_map) -> ()");
  m.def("silu_and_mul(Tensor! result, Tensor input) -> ()");
  m.def("silu_and_mul_with_clamp(Tensor! result, Tensor input, float limit, float alpha=1.0, float beta=0.0) -> ()");
  m.def("gelu_and_mul(Tensor! out, Tensor input) -> ()");
  m.def("gelu_tanh_and_mul(Tensor! out, Tensor input) -> ()");
  m.def("swigluoai_and_mul(Tensor! out, Tensor input, float alpha=1.702, float limit=7.0) -> ()");
  m.def("situ_and_mul(Tensor! out, Tensor input, float beta, float linear_beta) -> ()");
  m.def("swiglustep_and_mul(Tensor! out, Tensor input, float limit=7.0) -> ()");
  m.def("moe_sum(Tensor input, Tensor! output) -> ()");
  m.def("per_token_quant_int8(Tensor x) -> (Tensor, Tensor)");
  m.def("per_token_quant_fp8(Tensor x) -> (Tensor, Tensor)");
}
TORCH_LIBRARY_IMPL(sonar_amd, CUDA, m) {
  m.impl("moe_align_block_size", &moe_align_block_size);
  m.impl("silu_and_mul", &silu_and_mul);
  m.impl("silu_and_mul_with_clamp", &silu_and_mul_with_clamp);
  m.impl("gelu_and_mul", &gelu_and_mul);
  m.impl("gelu_tanh_and_mul", &gelu_tanh_and_mul);
  m.impl("swigluoai_and_mul", &swigluoai_and_mul);
  m.impl("situ_and_mul", &situ_and_mul);
  m.impl("swiglustep_and_mul", &swiglustep_and_mul);
  m.impl("moe_sum", &moe_sum);
  m.impl("per_token_quant_int8", &per_token_quant_int8);
  m.impl("per_token_quant_fp8", &per_token_quant_fp8);
}

TORCH_LIBRARY_FRAGMENT(_C, m) {
  m.def(
      "marlin_gemm(Tensor a, Tensor? c_or_none, Tensor b_q_weight, "
      "Tensor? b_bias_or_none,Tensor b_scales, "
      "Tensor? a_scales, Tensor? global_scale, Tensor? b_zeros_or_none, "
      "Tensor? "
      "g_idx_or_none, Tensor? perm_or_none, Tensor workspace, int b_type_id, "
      "SymInt size_m, SymInt size_n, SymInt size_k, bool is_k_full, "
      "bool use_atomic_add, bool use_fp32_reduce, bool is_zp_float) -> Tensor");
  // older name of the same op, still used by the reference's benchmark harness
  m.def(
      "gptq_marlin_gemm(Tensor a, Tensor? c_or_none, Tensor b_q_weight, "
      "Tensor? b_bias_or_none,Tensor b_scales, "
      "Tensor? a_scales, Tensor? global_scale, Tensor? b_zeros_or_none, "
      "Tensor? "
      "g_idx_or_none, Tensor? perm_or_none, Tensor workspace, int b_type_id, "
      "SymInt size_m, SymInt size_n, SymInt size_k, bool is_k_full, "
      "bool use_atomic_add, bool use_fp32_reduce, bool is_zp_float) -> Tensor");
  m.def(
      "gptq_marlin_repack(Tensor b_q_weight, Tensor perm, "
      "SymInt size_k, SymInt size_n, int num_bits, bool is_a_8bit) -> Tensor");
  m.def(
      "awq_marlin_repack(Tensor b_q_weight, SymInt size_k, "
      "SymInt size_n, int num_bits, bool is_a_8bit) -> Tensor");
  // not in the reference: Marlin order -> gfx950 streaming order, and cache control
  m.def("marlin_int4_fp8_preprocess(Tensor qweight, Tensor? qzeros_or_none, bool inplace) -> Tensor");
  m.def("marlin_to_gfx950(Tensor b_q_weight, SymInt size_k, SymInt size_n) -> Tensor");
  m.def("marlin_weight_cache_clear() -> int", &marlin_weight_cache_clear);
  m.def("marlin_weight_cache_invalidate(Tensor t) -> int", &marlin_weight_cache_invalidate);
}

TORCH_LIBRARY_IMPL(_C, CUDA, m) {
  m.impl("marlin_gemm", &marlin_gemm);
  m.impl("gptq_marlin_gemm", &marlin_gemm);
  m.impl("gptq_marlin_repack", &gptq_marlin_repack);
  m.impl("awq_marlin_repack", &awq_marlin_repack);
  m.impl("marlin_int4_fp8_preprocess", &marlin_int4_fp8_preprocess);
  m.impl("marlin_to_gfx950", &marlin_to_gfx950);
}

TORCH_LIBRARY_FRAGMENT(_moe_C, m) {
  m.def(
      "moe_wna16_marlin_gemm(Tensor! a, Tensor? c_or_none,"
      "Tensor! b_q_weight, Tensor? b_bias_or_none,"
      "Tensor! b_scales, Tensor? a_scales, Tensor? global_scale, Tensor? "
      "b_zeros_or_none,"
      "Tensor? g_idx_or_none, Tensor? perm_or_none, Tensor! workspace,"
      "Tensor sorted_token_ids,"
      "Tensor! expert_ids, Tensor! num_tokens_past_padded,"
      "Tensor! topk_weights, int moe_block_size, int top_k, "
      "bool mul_topk_weights, int b_type_id,"
      "int size_m, int size_n, int size_k,"
      "bool is_full_k, bool use_atomic_add,"
      "bool use_fp32_reduce, bool is_zp_float,"
      "int thread_k, int thread_n, int blocks_per_sm) -> Tensor");
}

TORCH_LIBRARY_IMPL(_moe_C, CUDA, m) { m.impl("moe_wna16_marlin_gemm", &moe_wna16_marlin_gemm); }

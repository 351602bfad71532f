// XLA FFI handlers over the C ABI of include/nvj_paged_attn.h, for registration
// with jax.ffi.register_ffi_target(..., platform="ROCM").
//
// This is the binding a JAX host (the reference's layers/attention.py:389-397 and
// :465-467 call sites) needs.  It only decodes buffers and attributes and calls
// the C ABI; no kernel code lives here.  It needs the XLA FFI headers that ship
// inside jaxlib (jax.ffi.include_dir()).  Those are NOT present in the image
// this library is developed in, so this file is built only when the build
// script finds them; it has not been compiled or run there.
//
//   hipcc -shared -fPIC -std=c++17 -I$(python -c "import jax.ffi; print(jax.ffi.include_dir())") \
//         -Iinclude nvj_xla_ffi.cc -L<dir of libnvj_paged_attn.so> -lnvj_paged_attn -o libnvj_xla_ffi.so
#include <hip/hip_runtime.h>

#include "nvj_paged_attn.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

ffi::Error to_error(int rc) {
  if (rc == NVJ_OK) return ffi::Error::Success();
  const ffi::ErrorCode code =
      rc == NVJ_ERR_LAUNCH ? ffi::ErrorCode::kInternal : ffi::ErrorCode::kInvalidArgument;
  return ffi::Error(code, nvj_error_string(rc));
}

// The handlers are typed for the bf16 caches of the Qwen3 models the reference runs; a float16
// cache binds the same way with F16 buffers and NVJ_DTYPE_F16.
int dtype_code(ffi::DataType t) { return t == ffi::DataType::F32 ? NVJ_DTYPE_F32 : NVJ_DTYPE_BF16; }

// operands: key, value [T, Hkv, D] (bf16 or f32), k_cache, v_cache [slots, Hkv, D] or
// [NB, bs, Hkv, D] bf16, slot_mapping [T] s32; results alias operands 2 and 3
// (input_output_aliases={2: 0, 3: 1}), so only the touched rows are written.
ffi::Error StoreKvcacheImpl(hipStream_t stream, ffi::AnyBuffer key, ffi::AnyBuffer value,
                            ffi::Buffer<ffi::DataType::BF16> k_cache_in,
                            ffi::Buffer<ffi::DataType::BF16> v_cache_in,
                            ffi::Buffer<ffi::DataType::S32> slot_mapping,
                            ffi::ResultBuffer<ffi::DataType::BF16> k_cache,
                            ffi::ResultBuffer<ffi::DataType::BF16> v_cache) {
  const auto kd = key.dimensions();
  if (kd.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "key must be [T,Hkv,D]");
  if (k_cache->untyped_data() != k_cache_in.untyped_data() ||
      v_cache->untyped_data() != v_cache_in.untyped_data())
    return ffi::Error(ffi::ErrorCode::kInvalidArgument,
                      "cache results must alias the cache operands (donate the caches)");
  const int64_t row = kd[1] * kd[2];
  const int64_t num_slots = row ? (int64_t)k_cache->element_count() / row : 0;
  return to_error(nvj_store_kvcache_launch(
      stream, key.untyped_data(), value.untyped_data(), k_cache->untyped_data(),
      v_cache->untyped_data(), slot_mapping.typed_data(), (int32_t)kd[0], (int32_t)kd[1],
      (int32_t)kd[2], num_slots, dtype_code(key.element_type()), dtype_code(value.element_type()),
      NVJ_DTYPE_BF16));
}

// operands: q [B, Hq, D], k_cache, v_cache [NB, bs, Hkv, D] bf16, block_tables [B, MB],
// context_lens [B] s32; attrs scale (f32), chunk (s32, 0 = balanced split, -1 = whole
// sequence per workgroup: the workspace result is then unused);
// results: out [B, Hq, D] bf16 and the workspace (u8, sized by
// nvj_paged_decode_workspace_bytes on the Python side so that XLA owns it).
ffi::Error PagedDecodeImpl(hipStream_t stream, ffi::Buffer<ffi::DataType::BF16> q,
                           ffi::Buffer<ffi::DataType::BF16> k_cache,
                           ffi::Buffer<ffi::DataType::BF16> v_cache,
                           ffi::Buffer<ffi::DataType::S32> block_tables,
                           ffi::Buffer<ffi::DataType::S32> context_lens, float scale,
                           int32_t chunk, ffi::ResultBuffer<ffi::DataType::BF16> out,
                           ffi::ResultBuffer<ffi::DataType::U8> workspace) {
  const auto qd = q.dimensions();
  const auto cd = k_cache.dimensions();
  const auto td = block_tables.dimensions();
  if (qd.size() != 3 || cd.size() != 4 || td.size() != 2)
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "bad operand ranks");
  return to_error(nvj_paged_decode_launch(
      stream, q.typed_data(), k_cache.typed_data(), v_cache.typed_data(),
      block_tables.typed_data(), context_lens.typed_data(), out->typed_data(),
      workspace->typed_data(), workspace->size_bytes(), (int32_t)qd[0], (int32_t)qd[1],
      (int32_t)cd[2], (int32_t)qd[2], (int32_t)cd[1], (int32_t)td[1], (int32_t)cd[0], scale,
      chunk, NVJ_DTYPE_BF16));
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    NvjStoreKvcache, StoreKvcacheImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::Buffer<ffi::DataType::BF16>>()
        .Arg<ffi::Buffer<ffi::DataType::BF16>>()
        .Arg<ffi::Buffer<ffi::DataType::S32>>()
        .Ret<ffi::Buffer<ffi::DataType::BF16>>()
        .Ret<ffi::Buffer<ffi::DataType::BF16>>(),
    {ffi::Traits::kCmdBufferCompatible});

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    NvjPagedDecode, PagedDecodeImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::Buffer<ffi::DataType::BF16>>()
        .Arg<ffi::Buffer<ffi::DataType::BF16>>()
        .Arg<ffi::Buffer<ffi::DataType::BF16>>()
        .Arg<ffi::Buffer<ffi::DataType::S32>>()
        .Arg<ffi::Buffer<ffi::DataType::S32>>()
        .Attr<float>("scale")
        .Attr<int32_t>("chunk")
        .Ret<ffi::Buffer<ffi::DataType::BF16>>()
        .Ret<ffi::Buffer<ffi::DataType::U8>>(),
    {ffi::Traits::kCmdBufferCompatible});

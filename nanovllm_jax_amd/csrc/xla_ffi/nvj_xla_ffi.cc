// XLA FFI handlers over the C ABI of include/nvj_paged_attn.h, for registration
// with jax.ffi.register_ffi_target(..., platform="ROCM").
//
// This is the binding a JAX host (the reference's layers/attention.py:389-397 and
// :465-467 call sites) needs.  It only decodes buffers and attributes and calls
// the C ABI; no kernel code lives here.  It needs the XLA FFI headers that ship
// inside jaxlib (jax.ffi.include_dir()).  Those are present neither in the image
// this library is developed in nor on its GPU machines (no jax, jaxlib or XLA
// headers on either), so this file is built only when the build script finds
// them: it has NEVER been compiled or run, and its parity is unpinned.
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

// Element type code of the C ABI for an XLA element type; -1 for anything the
// C ABI does not take (reported by the callers, never reinterpreted).
int dtype_code(ffi::DataType t) {
  switch (t) {
    case ffi::DataType::BF16: return NVJ_DTYPE_BF16;
    case ffi::DataType::F16: return NVJ_DTYPE_F16;
    case ffi::DataType::F32: return NVJ_DTYPE_F32;
    default: return -1;
  }
}

ffi::Error bad(const char* what) { return ffi::Error(ffi::ErrorCode::kInvalidArgument, what); }

// operands: key, value [T, Hkv, D] (cache dtype or f32), k_cache, v_cache [slots, Hkv, D] or
// [NB, bs, Hkv, D] (bf16 or f16, the model dtype), slot_mapping [T] s32; results alias
// operands 2 and 3 (input_output_aliases={2: 0, 3: 1}), as the reference's function
// returns the updated caches (layers/attention.py:42-77, rebound at :470-475), so only the
// touched rows are written.
ffi::Error StoreKvcacheImpl(hipStream_t stream, ffi::AnyBuffer key, ffi::AnyBuffer value,
                            ffi::AnyBuffer k_cache_in, ffi::AnyBuffer v_cache_in,
                            ffi::Buffer<ffi::DataType::S32> slot_mapping,
                            ffi::Result<ffi::AnyBuffer> k_cache,
                            ffi::Result<ffi::AnyBuffer> v_cache) {
  const auto kd = key.dimensions();
  if (kd.size() != 3) return bad("key must be [T,Hkv,D]");
  const int cache_code = dtype_code(k_cache->element_type());
  if (cache_code != NVJ_DTYPE_BF16 && cache_code != NVJ_DTYPE_F16)
    return bad("the KV cache must be bf16 or f16");
  if (v_cache->element_type() != k_cache->element_type() ||
      k_cache_in.element_type() != k_cache->element_type() ||
      v_cache_in.element_type() != k_cache->element_type())
    return bad("k_cache and v_cache must have one dtype");
  const int k_code = dtype_code(key.element_type()), v_code = dtype_code(value.element_type());
  if (k_code < 0 || v_code < 0) return bad("key / value must be bf16, f16 or f32");
  if (k_cache->untyped_data() != k_cache_in.untyped_data() ||
      v_cache->untyped_data() != v_cache_in.untyped_data())
    return bad("cache results must alias the cache operands (donate the caches)");
  const int64_t row = kd[1] * kd[2];
  const int64_t num_slots = row ? (int64_t)k_cache->element_count() / row : 0;
  return to_error(nvj_store_kvcache_launch(
      stream, key.untyped_data(), value.untyped_data(), k_cache->untyped_data(),
      v_cache->untyped_data(), slot_mapping.typed_data(), (int32_t)kd[0], (int32_t)kd[1],
      (int32_t)kd[2], num_slots, k_code, v_code, cache_code));
}

// operands: q [B, Hq, D], k_cache, v_cache [NB, bs, Hkv, D] (one dtype, bf16 or f16),
// block_tables [B, MB], context_lens [B] s32; attrs scale (f32), chunk (s32, 0 = balanced
// split, -1 = whole sequence per workgroup: the workspace result is then unused);
// results: out [B, Hq, D] in q's dtype and the workspace (u8, sized by
// nvj_paged_decode_workspace_bytes on the Python side so that XLA owns it).  XLA hands
// over the workspace uninitialised.  The balanced split therefore keeps only its
// partials there and takes its counters from the library's own region (zero between
// calls by invariant), which makes the call a single launch; the executables of one
// process must then not run decode calls on two streams of one GPU at the same time
// (XLA's GPU client runs compute on one stream per device).  The attr
// library_counters = 0 gives up the invariant instead: the whole workspace goes through
// nvj_paged_decode_launch, which clears its counters with a small kernel of its own.
ffi::Error PagedDecodeImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::AnyBuffer k_cache,
                           ffi::AnyBuffer v_cache, ffi::Buffer<ffi::DataType::S32> block_tables,
                           ffi::Buffer<ffi::DataType::S32> context_lens, float scale,
                           int32_t chunk, int32_t library_counters,
                           ffi::Result<ffi::AnyBuffer> out,
                           ffi::ResultBuffer<ffi::DataType::U8> workspace) {
  const auto qd = q.dimensions();
  const auto cd = k_cache.dimensions();
  const auto td = block_tables.dimensions();
  if (qd.size() != 3 || cd.size() != 4 || td.size() != 2) return bad("bad operand ranks");
  const int code = dtype_code(q.element_type());
  if (code != NVJ_DTYPE_BF16 && code != NVJ_DTYPE_F16) return bad("q must be bf16 or f16");
  if (k_cache.element_type() != q.element_type() || v_cache.element_type() != q.element_type() ||
      out->element_type() != q.element_type())
    return bad("q, k_cache, v_cache and out must have one dtype");
  if (chunk == 0 && library_counters != 0)
    return to_error(nvj_paged_decode_launch_counters(
        stream, q.untyped_data(), k_cache.untyped_data(), v_cache.untyped_data(),
        block_tables.typed_data(), context_lens.typed_data(), out->untyped_data(),
        workspace->typed_data(), workspace->size_bytes(), nullptr, 0, (int32_t)qd[0],
        (int32_t)qd[1], (int32_t)cd[2], (int32_t)qd[2], (int32_t)cd[1], (int32_t)td[1],
        (int32_t)cd[0], scale, code, NVJ_PHASE_SPLITK));
  return to_error(nvj_paged_decode_launch(
      stream, q.untyped_data(), k_cache.untyped_data(), v_cache.untyped_data(),
      block_tables.typed_data(), context_lens.typed_data(), out->untyped_data(),
      workspace->typed_data(), workspace->size_bytes(), (int32_t)qd[0], (int32_t)qd[1],
      (int32_t)cd[2], (int32_t)qd[2], (int32_t)cd[1], (int32_t)td[1], (int32_t)cd[0], scale,
      chunk, code));
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    NvjStoreKvcache, StoreKvcacheImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::Buffer<ffi::DataType::S32>>()
        .Ret<ffi::AnyBuffer>()
        .Ret<ffi::AnyBuffer>(),
    {ffi::Traits::kCmdBufferCompatible});

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    NvjPagedDecode, PagedDecodeImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::Buffer<ffi::DataType::S32>>()
        .Arg<ffi::Buffer<ffi::DataType::S32>>()
        .Attr<float>("scale")
        .Attr<int32_t>("chunk")
        .Attr<int32_t>("library_counters")
        .Ret<ffi::AnyBuffer>()
        .Ret<ffi::Buffer<ffi::DataType::U8>>(),
    {ffi::Traits::kCmdBufferCompatible});

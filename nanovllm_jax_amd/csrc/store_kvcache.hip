// KV-cache store for gfx950: scatter the new K/V rows of a step through
// slot_mapping into the block-paged cache, in place.
//
// Stands in for store_kv_to_cache (layers/attention.py:42-77 of the
// reference): cast to the cache dtype (:70-71), then cache[slot] = row for
// every in-range slot (:74-75).  Out-of-range slots are dropped, negative
// slots are skipped.  HBM-bound byte shuffling: every lane moves one 16-byte
// piece of a row (8 cache elements, bf16 or IEEE half), reading either 16
// bytes (source already in the cache's type) or 32 bytes (f32 source, rounded
// to nearest even here).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch.h"
#include "nvj_paged_attn.h"

namespace {

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet.  Integer
// arithmetic so the result is bit-identical on every path.
__device__ __forceinline__ uint32_t f32_to_bf16_rne(uint32_t u) {
  uint32_t r = (u + (((u >> 16) & 1u) + 0x7FFFu)) >> 16;
  const bool is_nan = (u & 0x7FFFFFFFu) > 0x7F800000u;
  return is_nan ? ((u >> 16) | 0x0040u) : r;
}

// fp32 -> IEEE half bits, round to nearest even (the hardware conversion).
__device__ __forceinline__ uint32_t f32_to_f16_rne(uint32_t u) {
  const _Float16 h = (_Float16)__uint_as_float(u);
  return (uint32_t)__builtin_bit_cast(uint16_t, h);
}

// One piece of a source row as 8 cache elements.  F32: the source is float32
// and is rounded to the cache's type (CF16: IEEE half, else bf16); otherwise
// the source already has the cache's type and is copied.
template <bool F32, bool CF16>
__device__ __forceinline__ uint4 load_piece_as_cache_type(const void* src, int64_t piece) {
  if constexpr (!F32) {
    return reinterpret_cast<const uint4*>(src)[piece];
  } else {
    const uint4* p = reinterpret_cast<const uint4*>(src) + 2 * piece;
    const uint4 a = p[0], b = p[1];
    auto cvt = [](uint32_t u) { return CF16 ? f32_to_f16_rne(u) : f32_to_bf16_rne(u); };
    uint4 o;
    o.x = cvt(a.x) | (cvt(a.y) << 16);
    o.y = cvt(a.z) | (cvt(a.w) << 16);
    o.z = cvt(b.x) | (cvt(b.y) << 16);
    o.w = cvt(b.z) | (cvt(b.w) << 16);
    return o;
  }
}

// One lane per 16-byte piece of one token row, for K and V both.
// pieces_per_row = num_kv_heads * head_dim / 8.
template <bool KF32, bool VF32, bool CF16>
__global__ __launch_bounds__(256) void store_kvcache_kernel(
    const void* __restrict__ key, const void* __restrict__ value,
    uint4* __restrict__ k_cache, uint4* __restrict__ v_cache,
    const int32_t* __restrict__ slot_mapping, int num_tokens,
    int pieces_per_row, int64_t num_slots) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)num_tokens * pieces_per_row;
  if (gid >= total) return;
  const int token = (int)(gid / pieces_per_row);
  const int piece = (int)(gid - (int64_t)token * pieces_per_row);
  const int64_t slot = slot_mapping[token];
  if (slot < 0 || slot >= num_slots) return;
  const uint4 kb = load_piece_as_cache_type<KF32, CF16>(key, gid);
  const uint4 vb = load_piece_as_cache_type<VF32, CF16>(value, gid);
  const int64_t dst = slot * pieces_per_row + piece;
  k_cache[dst] = kb;
  v_cache[dst] = vb;
}

}  // namespace

extern "C" int nvj_store_kvcache_launch(void* stream, const void* key, const void* value,
                                        void* k_cache, void* v_cache,
                                        const int32_t* slot_mapping, int32_t num_tokens,
                                        int32_t num_kv_heads, int32_t head_dim,
                                        int64_t num_slots, int32_t k_dtype,
                                        int32_t v_dtype, int32_t cache_dtype) {
  if (num_tokens < 0 || num_kv_heads <= 0 || head_dim <= 0 || num_slots < 0)
    return NVJ_ERR_BAD_SHAPE;
  if (cache_dtype != NVJ_DTYPE_BF16 && cache_dtype != NVJ_DTYPE_F16) return NVJ_ERR_BAD_DTYPE;
  // a source is float32 (rounded here) or already has the cache's type
  if ((k_dtype != cache_dtype && k_dtype != NVJ_DTYPE_F32) ||
      (v_dtype != cache_dtype && v_dtype != NVJ_DTYPE_F32))
    return NVJ_ERR_BAD_DTYPE;
  const int64_t row = (int64_t)num_kv_heads * head_dim;
  if (row % 8 != 0 || row / 8 > INT32_MAX) return NVJ_ERR_UNSUPPORTED;
  if (num_tokens == 0) return NVJ_OK;
  if (!key || !value || !k_cache || !v_cache || !slot_mapping) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(key) | reinterpret_cast<uintptr_t>(value) |
       reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache)) & 15u)
    return NVJ_ERR_ALIGNMENT;
  const int pieces = (int)(row / 8);
  const int64_t total = (int64_t)num_tokens * pieces;
  const int64_t blocks = (total + 255) / 256;
  if (blocks > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((unsigned)blocks), block(256);
  uint4* kc = static_cast<uint4*>(k_cache);
  uint4* vc = static_cast<uint4*>(v_cache);
  const bool kf = k_dtype == NVJ_DTYPE_F32, vf = v_dtype == NVJ_DTYPE_F32;
  const bool cf16 = cache_dtype == NVJ_DTYPE_F16;
  hipError_t rc;
#define NVJ_LAUNCH_STORE(KF, VF, CF)                                                      \
  rc = nvj::launch(store_kvcache_kernel<KF, VF, CF>, grid, block, s, key, value, kc, vc, \
                   slot_mapping, num_tokens, pieces, num_slots)
  switch ((kf ? 4 : 0) | (vf ? 2 : 0) | (cf16 ? 1 : 0)) {
    case 0: NVJ_LAUNCH_STORE(false, false, false); break;   // copies: the type does not matter
    case 1: NVJ_LAUNCH_STORE(false, false, false); break;
    case 2: NVJ_LAUNCH_STORE(false, true, false); break;
    case 3: NVJ_LAUNCH_STORE(false, true, true); break;
    case 4: NVJ_LAUNCH_STORE(true, false, false); break;
    case 5: NVJ_LAUNCH_STORE(true, false, true); break;
    case 6: NVJ_LAUNCH_STORE(true, true, false); break;
    default: NVJ_LAUNCH_STORE(true, true, true); break;
  }
#undef NVJ_LAUNCH_STORE
  return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

// KV-cache store for gfx950: scatter the new K/V rows of a step through
// slot_mapping into the block-paged cache, in place.
//
// Stands in for store_kv_to_cache (layers/attention.py:42-77 of the
// reference): cast to the cache dtype (:70-71), then cache[slot] = row for
// every in-range slot (:74-75).  Out-of-range slots are dropped, negative
// slots are skipped.  HBM-bound byte shuffling: every lane moves one 16-byte
// piece of a row (8 bf16), reading either 16 bytes (bf16 source) or 32 bytes
// (f32 source, rounded to nearest even here).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nvj_paged_attn.h"

namespace {

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet.  Integer
// arithmetic so the result is bit-identical on every path.
__device__ __forceinline__ uint32_t f32_to_bf16_rne(uint32_t u) {
  uint32_t r = (u + (((u >> 16) & 1u) + 0x7FFFu)) >> 16;
  const bool is_nan = (u & 0x7FFFFFFFu) > 0x7F800000u;
  return is_nan ? ((u >> 16) | 0x0040u) : r;
}

template <bool F32>
__device__ __forceinline__ uint4 load_piece_as_bf16(const void* src, int64_t piece) {
  if constexpr (!F32) {
    return reinterpret_cast<const uint4*>(src)[piece];
  } else {
    const uint4* p = reinterpret_cast<const uint4*>(src) + 2 * piece;
    const uint4 a = p[0], b = p[1];
    uint4 o;
    o.x = f32_to_bf16_rne(a.x) | (f32_to_bf16_rne(a.y) << 16);
    o.y = f32_to_bf16_rne(a.z) | (f32_to_bf16_rne(a.w) << 16);
    o.z = f32_to_bf16_rne(b.x) | (f32_to_bf16_rne(b.y) << 16);
    o.w = f32_to_bf16_rne(b.z) | (f32_to_bf16_rne(b.w) << 16);
    return o;
  }
}

// One lane per 16-byte piece of one token row, for K and V both.
// pieces_per_row = num_kv_heads * head_dim / 8.
template <bool KF32, bool VF32>
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
  const uint4 kb = load_piece_as_bf16<KF32>(key, gid);
  const uint4 vb = load_piece_as_bf16<VF32>(value, gid);
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
                                        int32_t v_dtype) {
  if (num_tokens < 0 || num_kv_heads <= 0 || head_dim <= 0 || num_slots < 0)
    return NVJ_ERR_BAD_SHAPE;
  if ((k_dtype != NVJ_DTYPE_BF16 && k_dtype != NVJ_DTYPE_F32) ||
      (v_dtype != NVJ_DTYPE_BF16 && v_dtype != NVJ_DTYPE_F32))
    return NVJ_ERR_BAD_DTYPE;
  const int64_t row = (int64_t)num_kv_heads * head_dim;
  if (row % 8 != 0 || row / 8 > INT32_MAX) return NVJ_ERR_UNSUPPORTED;
  if (num_tokens == 0) return NVJ_OK;
  if (!key || !value || !k_cache || !v_cache || !slot_mapping) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(key) | reinterpret_cast<uintptr_t>(value) |
       reinterpret_cast<uintptr_t>(k_cache) | reinterpret_cast<uintptr_t>(v_cache)) & 15u)
    return NVJ_ERR_BAD_SHAPE;
  const int pieces = (int)(row / 8);
  const int64_t total = (int64_t)num_tokens * pieces;
  const int64_t blocks = (total + 255) / 256;
  if (blocks > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((unsigned)blocks), block(256);
  uint4* kc = static_cast<uint4*>(k_cache);
  uint4* vc = static_cast<uint4*>(v_cache);
  const bool kf = k_dtype == NVJ_DTYPE_F32, vf = v_dtype == NVJ_DTYPE_F32;
  if (kf && vf)
    store_kvcache_kernel<true, true><<<grid, block, 0, s>>>(key, value, kc, vc, slot_mapping,
                                                            num_tokens, pieces, num_slots);
  else if (kf)
    store_kvcache_kernel<true, false><<<grid, block, 0, s>>>(key, value, kc, vc, slot_mapping,
                                                             num_tokens, pieces, num_slots);
  else if (vf)
    store_kvcache_kernel<false, true><<<grid, block, 0, s>>>(key, value, kc, vc, slot_mapping,
                                                             num_tokens, pieces, num_slots);
  else
    store_kvcache_kernel<false, false><<<grid, block, 0, s>>>(key, value, kc, vc, slot_mapping,
                                                              num_tokens, pieces, num_slots);
  return hipGetLastError() == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

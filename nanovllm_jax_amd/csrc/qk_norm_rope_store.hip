// Fused per-head QK-RMSNorm + rotary embedding + KV-cache store for gfx950.
//
// One launch replaces the chain the reference runs between the QKV projection
// and the attention call of a decode (or prefill) step:
//   q, k = q_norm(q), k_norm(k)        models/qwen3.py:157-160, layers/layernorm.py:31-48
//   q, k = rotary_emb(positions, q, k) models/qwen3.py:163, layers/rotary_embedding.py:13-37,96-106
//   q -> cache dtype                   layers/attention.py:386-387
//   store_kv_to_cache(k, v, ...)       layers/attention.py:42-77 (cast at :70-71)
// It reads the packed QKV projection output once and writes q (bf16) plus the
// K and V cache rows; nothing else touches HBM.
//
// One wave64 per (token, head).  Lane l holds elements l and l + 64 of the
// 128-wide head, which is exactly one rotary pair, so the rotation needs no
// cross-lane traffic; the mean of squares is a 6-step xor butterfly.  The
// arithmetic is a fixed sequence of IEEE fp32 operations (no contraction, no
// approximate rsqrt) so that a CPU restatement reproduces it bit for bit:
//   s_l   = fma(x2, x2, x1 * x1)            (fp32 values of the bf16 inputs)
//   s_l  += s_(l ^ m)  for m = 32, 16, 8, 4, 2, 1
//   r     = 1 / sqrt(s / 128 + eps)
//   n_i   = bf16(x_i * r * w_i)             (cast back to the input dtype)
//   y1    = n1 * cos - n2 * sin,  y2 = n2 * cos + n1 * sin   (fp32)
//   out   = bf16(y)                         (round to nearest even)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch.h"
#include "nvj_paged_attn.h"

namespace {

constexpr int kHeadDim = 128;
constexpr int kHalf = 64;

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  return (uint16_t)((u + (((u >> 16) & 1u) + 0x7FFFu)) >> 16);
}

// grid.x = ceil(num_tokens * heads_total / 4), block = 256 (4 waves).
__global__ __launch_bounds__(256) void qk_norm_rope_store_kernel(
    const uint16_t* __restrict__ qkv, int64_t qkv_row_stride,   // [T, >= (Hq+2Hkv)*128] bf16
    const int32_t* __restrict__ positions,                       // [T]
    const float* __restrict__ cos_sin, int max_position,         // [max_position, 128]: cos | sin
    const float* __restrict__ q_weight, const float* __restrict__ k_weight,  // [128] or null
    float eps, const int32_t* __restrict__ slot_mapping,         // [T]
    uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,          // [num_slots, Hkv, 128]
    uint16_t* __restrict__ q_out,                                 // [T, Hq, 128]
    int num_tokens, int num_heads, int num_kv_heads, int64_t num_slots) {
#pragma clang fp contract(off)
  const int heads_total = num_heads + 2 * num_kv_heads;
  const int64_t unit = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= (int64_t)num_tokens * heads_total) return;
  const int token = (int)(unit / heads_total);
  const int head = (int)(unit - (int64_t)token * heads_total);
  const int lane = threadIdx.x & 63;
  const uint16_t* src = qkv + (int64_t)token * qkv_row_stride + (int64_t)head * kHeadDim;

  const bool is_q = head < num_heads;
  const bool is_k = !is_q && head < num_heads + num_kv_heads;
  int64_t slot = 0;
  if (!is_q) {
    slot = slot_mapping[token];
    if (slot < 0 || slot >= num_slots) return;   // skipped / dropped token
  }
  if (!is_q && !is_k) {   // V: plain row copy into the cache
    const int kvh = head - num_heads - num_kv_heads;
    const uint32_t* s32 = reinterpret_cast<const uint32_t*>(src);
    uint32_t* d32 = reinterpret_cast<uint32_t*>(v_cache + (slot * num_kv_heads + kvh) * kHeadDim);
    d32[lane] = s32[lane];
    return;
  }

  float x1 = bf16_to_f32(src[lane]);
  float x2 = bf16_to_f32(src[lane + kHalf]);
  const float* w = is_q ? q_weight : k_weight;
  if (w != nullptr) {
    float s = __builtin_fmaf(x2, x2, x1 * x1);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
    const float r = 1.0f / __builtin_sqrtf(s * (1.0f / kHeadDim) + eps);
    x1 = bf16_to_f32(f32_to_bf16_rne(x1 * r * w[lane]));
    x2 = bf16_to_f32(f32_to_bf16_rne(x2 * r * w[lane + kHalf]));
  }
  int pos = positions[token];
  pos = min(max(pos, 0), max_position - 1);
  const float c = cos_sin[(int64_t)pos * kHeadDim + lane];
  const float sn = cos_sin[(int64_t)pos * kHeadDim + kHalf + lane];
  const float y1 = x1 * c - x2 * sn;
  const float y2 = x2 * c + x1 * sn;
  uint16_t* dst;
  if (is_q) {
    dst = q_out + ((int64_t)token * num_heads + head) * kHeadDim;
  } else {
    dst = k_cache + (slot * num_kv_heads + (head - num_heads)) * kHeadDim;
  }
  dst[lane] = f32_to_bf16_rne(y1);
  dst[lane + kHalf] = f32_to_bf16_rne(y2);
}

}  // namespace

extern "C" int nvj_qk_norm_rope_store_launch(void* stream, const void* qkv, int64_t qkv_row_stride,
                                             const int32_t* positions, const float* cos_sin_cache,
                                             int32_t max_position, const float* q_norm_weight,
                                             const float* k_norm_weight, float eps,
                                             const int32_t* slot_mapping, void* k_cache,
                                             void* v_cache, void* q_out, int32_t num_tokens,
                                             int32_t num_heads, int32_t num_kv_heads,
                                             int32_t head_dim, int64_t num_slots) {
  if (num_tokens < 0 || num_heads <= 0 || num_kv_heads <= 0 || max_position <= 0 || num_slots < 0)
    return NVJ_ERR_BAD_SHAPE;
  if (head_dim != kHeadDim) return NVJ_ERR_UNSUPPORTED;
  const int64_t heads_total = (int64_t)num_heads + 2 * (int64_t)num_kv_heads;
  if (qkv_row_stride < heads_total * kHeadDim || (qkv_row_stride & 1)) return NVJ_ERR_BAD_SHAPE;
  if (num_tokens == 0) return NVJ_OK;
  if (!qkv || !positions || !cos_sin_cache || !slot_mapping || !k_cache || !v_cache || !q_out)
    return NVJ_ERR_NULL_POINTER;
  if ((q_norm_weight == nullptr) != (k_norm_weight == nullptr)) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(k_cache) |
       reinterpret_cast<uintptr_t>(v_cache) | reinterpret_cast<uintptr_t>(q_out)) & 3u)
    return NVJ_ERR_ALIGNMENT;
  const int64_t units = (int64_t)num_tokens * heads_total;
  const int64_t blocks = (units + 3) / 4;
  if (blocks > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  const hipError_t rc = nvj::launch(
      qk_norm_rope_store_kernel, dim3((unsigned)blocks), dim3(256),
      static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(qkv), qkv_row_stride, positions, cos_sin_cache, max_position,
      q_norm_weight, k_norm_weight, eps, slot_mapping, static_cast<uint16_t*>(k_cache),
      static_cast<uint16_t*>(v_cache), static_cast<uint16_t*>(q_out), num_tokens, num_heads,
      num_kv_heads, num_slots);
  return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

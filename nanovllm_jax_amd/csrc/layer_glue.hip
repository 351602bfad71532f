// The two element-wise stages that sit between the projections of a decoder
// layer, each as one launch for gfx950:
//   * RMSNorm, optionally fused with the residual add: RMSNorm._rms_forward and
//     RMSNorm._add_rms_forward (layers/layernorm.py:31-48 and :50-79 of the
//     reference), as called at models/qwen3.py:305-313;
//   * SiLU(gate) * up: SiluAndMul.__call__ (layers/activation.py:22-33).
// Both are HBM/launch-latency bound row operations (one wave64 per token row);
// in a decode step they replace chains of 2-5 framework kernels per call.
//
// RMSNorm arithmetic is a fixed sequence of IEEE fp32 operations (no
// contraction, no approximate rsqrt) so that a CPU restatement reproduces it bit
// for bit.  With the row cut into 16-byte pieces of 8 bf16, lane l owns pieces
// l, l + 64, l + 128, ...:
//   s_i    = f32(x_i) + f32(residual_i)         (or f32(x_i) without a residual)
//   res_i  = bf16(s_i)                           (the new residual, layernorm.py:68-69)
//   a_l    = ((0 + s*s) + s*s) + ...             over the lane's elements in row order
//   a_l   += a_(l ^ m)  for m = 32, 16, 8, 4, 2, 1
//   r      = 1 / sqrt(a * (1 / hidden) + eps)    (mean of the unrounded sums, :72-73)
//   y_i    = bf16((s_i * r) * w_i)               (:76)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch.h"
#include "nvj_paged_attn.h"

namespace {

constexpr int kMaxPiecesPerLane = 16;   // hidden <= 64 * 8 * 16 = 8192

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }

__device__ __forceinline__ uint32_t f32_to_bf16_rne(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x0040u;
  return (u + (((u >> 16) & 1u) + 0x7FFFu)) >> 16;
}
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  return f32_to_bf16_rne(lo) | (f32_to_bf16_rne(hi) << 16);
}

__device__ __forceinline__ void unpack8(const uint4& p, float (&f)[8]) {
  f[0] = bf16_lo(p.x); f[1] = bf16_hi(p.x);
  f[2] = bf16_lo(p.y); f[3] = bf16_hi(p.y);
  f[4] = bf16_lo(p.z); f[5] = bf16_hi(p.z);
  f[6] = bf16_lo(p.w); f[7] = bf16_hi(p.w);
}

// grid.x = ceil(num_tokens / 4), block = 256 (4 waves, one token row each).
// PIECES = 16-byte pieces per lane, a compile-time bound so the row stays in
// registers between the two passes.
template <int PIECES, bool RESIDUAL>
__global__ __launch_bounds__(256) void add_rms_norm_kernel(
    const uint4* __restrict__ x, const uint4* residual, const float* __restrict__ weight,
    float eps, uint4* __restrict__ y, uint4* residual_out, int num_tokens, int row_pieces) {
#pragma clang fp contract(off)
  const int token = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (token >= num_tokens) return;
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)token * row_pieces;

  // every load of the row is issued before the first store: residual_out may be
  // the residual buffer itself, so a store would otherwise fence the loads
  // that follow it
  uint4 xv[PIECES], rv[PIECES];
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int p = lane + 64 * j;
    if (p < row_pieces) {
      xv[j] = x[row + p];
      if (RESIDUAL) rv[j] = residual[row + p];
    }
  }
  // short rows: the weights too, ahead of the reduction
  constexpr bool kEarlyWeights = PIECES <= 2;
  float4 wv[kEarlyWeights ? PIECES : 1][2];
  if (kEarlyWeights) {
#pragma unroll
    for (int j = 0; j < PIECES; ++j) {
      const int p = lane + 64 * j;
      if (p < row_pieces) {
        wv[j][0] = reinterpret_cast<const float4*>(weight)[2 * p];
        wv[j][1] = reinterpret_cast<const float4*>(weight)[2 * p + 1];
      }
    }
  }

  float s[PIECES][8];
  float a = 0.f;
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int p = lane + 64 * j;
    if (p < row_pieces) {
      unpack8(xv[j], s[j]);
      if (RESIDUAL) {
        float rs[8];
        unpack8(rv[j], rs);
#pragma unroll
        for (int e = 0; e < 8; ++e) s[j][e] = s[j][e] + rs[e];
        uint4 o;
        o.x = pack2(s[j][0], s[j][1]);
        o.y = pack2(s[j][2], s[j][3]);
        o.z = pack2(s[j][4], s[j][5]);
        o.w = pack2(s[j][6], s[j][7]);
        residual_out[row + p] = o;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) a = a + s[j][e] * s[j][e];
    }
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) a += __shfl_xor(a, m, 64);
  const float r = 1.0f / __builtin_sqrtf(a * (1.0f / (float)(row_pieces * 8)) + eps);
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int p = lane + 64 * j;
    if (p < row_pieces) {
      const float4 w0 =
          kEarlyWeights ? wv[kEarlyWeights ? j : 0][0] : reinterpret_cast<const float4*>(weight)[2 * p];
      const float4 w1 = kEarlyWeights ? wv[kEarlyWeights ? j : 0][1]
                                      : reinterpret_cast<const float4*>(weight)[2 * p + 1];
      uint4 o;
      o.x = pack2(s[j][0] * r * w0.x, s[j][1] * r * w0.y);
      o.y = pack2(s[j][2] * r * w0.z, s[j][3] * r * w0.w);
      o.z = pack2(s[j][4] * r * w1.x, s[j][5] * r * w1.y);
      o.w = pack2(s[j][6] * r * w1.z, s[j][7] * r * w1.w);
      y[row + p] = o;
    }
  }
}

// SiLU(gate) * up in fp32 from the bf16 inputs, rounded once to bf16.
// grid.x covers num_tokens * (intermediate / 8) pieces, one per lane.
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const uint4* __restrict__ x,
                                                           int64_t x_row_pieces,
                                                           uint4* __restrict__ y, int num_tokens,
                                                           int out_pieces) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)num_tokens * out_pieces) return;
  const int token = (int)(i / out_pieces);
  const int p = (int)(i - (int64_t)token * out_pieces);
  float g[8], u[8];
  unpack8(x[(int64_t)token * x_row_pieces + p], g);
  unpack8(x[(int64_t)token * x_row_pieces + out_pieces + p], u);
  float o[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = g[e] / (1.0f + expf(-g[e])) * u[e];
  uint4 out;
  out.x = pack2(o[0], o[1]);
  out.y = pack2(o[2], o[3]);
  out.z = pack2(o[4], o[5]);
  out.w = pack2(o[6], o[7]);
  y[i] = out;
}

template <int PIECES>
hipError_t launch_add_rms_norm(hipStream_t stream, const uint4* x, const uint4* residual,
                         const float* weight, float eps, uint4* y, uint4* residual_out,
                         int num_tokens, int row_pieces) {
  const dim3 grid((unsigned)((num_tokens + 3) / 4)), block(256);
  if (residual != nullptr)
    return nvj::launch(add_rms_norm_kernel<PIECES, true>, grid, block, stream, x, residual, weight,
                       eps, y, residual_out, num_tokens, row_pieces);
  return nvj::launch(add_rms_norm_kernel<PIECES, false>, grid, block, stream, x, nullptr, weight,
                     eps, y, nullptr, num_tokens, row_pieces);
}

}  // namespace

extern "C" int nvj_add_rms_norm_launch(void* stream, const void* x, const void* residual,
                                       const float* weight, float eps, void* y,
                                       void* residual_out, int32_t num_tokens, int32_t hidden) {
  if (num_tokens < 0 || hidden <= 0) return NVJ_ERR_BAD_SHAPE;
  if (hidden % 8 != 0 || hidden > 64 * 8 * kMaxPiecesPerLane) return NVJ_ERR_UNSUPPORTED;
  if (num_tokens == 0) return NVJ_OK;
  if (!x || !weight || !y) return NVJ_ERR_NULL_POINTER;
  if ((residual == nullptr) != (residual_out == nullptr)) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(residual) |
       reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(y) |
       reinterpret_cast<uintptr_t>(residual_out)) & 15u)
    return NVJ_ERR_ALIGNMENT;
  const int row_pieces = hidden / 8;
  const int per_lane = (row_pieces + 63) / 64;
  const auto s = static_cast<hipStream_t>(stream);
  const auto xp = static_cast<const uint4*>(x);
  const auto rp = static_cast<const uint4*>(residual);
  const auto yp = static_cast<uint4*>(y);
  const auto op = static_cast<uint4*>(residual_out);
  hipError_t rc;
  if (per_lane <= 1) rc = launch_add_rms_norm<1>(s, xp, rp, weight, eps, yp, op, num_tokens, row_pieces);
  else if (per_lane <= 2) rc = launch_add_rms_norm<2>(s, xp, rp, weight, eps, yp, op, num_tokens, row_pieces);
  else if (per_lane <= 4) rc = launch_add_rms_norm<4>(s, xp, rp, weight, eps, yp, op, num_tokens, row_pieces);
  else if (per_lane <= 8) rc = launch_add_rms_norm<8>(s, xp, rp, weight, eps, yp, op, num_tokens, row_pieces);
  else rc = launch_add_rms_norm<16>(s, xp, rp, weight, eps, yp, op, num_tokens, row_pieces);
  return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

extern "C" int nvj_silu_and_mul_launch(void* stream, const void* x, int64_t x_row_stride, void* y,
                                       int32_t num_tokens, int32_t intermediate) {
  if (num_tokens < 0 || intermediate <= 0) return NVJ_ERR_BAD_SHAPE;
  if (intermediate % 8 != 0) return NVJ_ERR_UNSUPPORTED;
  if (x_row_stride < 2 * (int64_t)intermediate || x_row_stride % 8 != 0) return NVJ_ERR_BAD_SHAPE;
  if (num_tokens == 0) return NVJ_OK;
  if (!x || !y) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u)
    return NVJ_ERR_ALIGNMENT;
  const int out_pieces = intermediate / 8;
  const int64_t blocks = ((int64_t)num_tokens * out_pieces + 255) / 256;
  if (blocks > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  const hipError_t rc = nvj::launch(
      silu_and_mul_kernel, dim3((unsigned)blocks), dim3(256), static_cast<hipStream_t>(stream),
      static_cast<const uint4*>(x), x_row_stride / 8, static_cast<uint4*>(y), num_tokens,
      out_pieces);
  return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

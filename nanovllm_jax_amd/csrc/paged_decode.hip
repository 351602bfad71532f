// Split-K paged decode attention for gfx950 (CDNA4, wave64) and its combine pass.
//
// Stands in for paged_attention -> paged_decode_attention_vectorized
// (layers/pallas_attention.py:465-507, :146-238 of the reference) and for the
// gather + dot_product_attention fallback (layers/attention.py:399-434).
//
// Work split.  One workgroup handles `chunk` consecutive positions of one
// sequence for NW KV heads at once, one wave per KV head, so the workgroup as
// a whole streams whole 2 KiB cache rows (all heads of a position are
// contiguous in the [page, position, head, dim] layout).  A wave owns the G
// query heads of its KV head, so every K/V byte is fetched once per group.
//
// Inner step = 32 positions of one page:
//   * K: 8 x 16-byte loads per lane, quarter-wave = one 256-byte (position,
//     head) row; staged through a wave-private, padded LDS tile and read back
//     in the MFMA A-operand layout (lane = position, 8 consecutive dims).
//   * S^T[pos, qhead] = K . Q^T with v_mfma_f32_16x16x32_bf16 (query heads
//     padded to 16 columns, held in registers for the whole chunk).
//   * fp32 online softmax on the accumulator layout (lane = query head,
//     4 positions per tile), running max shared across the 4 lane groups.
//   * V: 8 x 16-byte loads per lane straight from HBM, one per position the
//     lane's P^T operand holds, transposed inside the lane with v_perm_b32
//     into 8 A operands (lane = 8 dims x 8 positions), so no LDS for V.
//   * O^T[dim, qhead] += V^T . P^T with 8 MFMAs.
// Loads for step i+1 are issued before the arithmetic of step i.
//
// The partial (unnormalised O, running max, running sum) of every chunk goes
// to the workspace; the combine kernel merges the chunks of a sequence.  A
// sequence that fits one chunk is written directly.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nvj_paged_attn.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kHeadDim = 128;
constexpr int kStep = 32;            // positions per inner step
constexpr int kRowPieces = 16;       // 16-byte pieces per (position, head) row
constexpr int kLdsRowPieces = 17;    // padded LDS row, in 16-byte pieces
constexpr float kNegBig = -1.0e30f;  // stands for -inf without inf-inf hazards
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  bf16x2 p = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, p);
}

__device__ __forceinline__ float wave_xor_max(float x, int mask) {
  return fmaxf(x, __shfl_xor(x, mask, 64));
}

// Byte offset of load slot `x` (position within the step) for this lane, as a
// 32-bit quantity: a step never leaves its page, so it is below
// block_size * row_bytes.  TAIL steps clamp the slot to the last live position
// so nothing at or beyond the context length is ever read.
template <bool TAIL>
__device__ __forceinline__ uint32_t slot_offset(int x, int last, uint32_t row_bytes,
                                                uint32_t lane_bytes) {
  if constexpr (TAIL) x = min(x, last);
  return (uint32_t)x * row_bytes + lane_bytes;
}

// K/V are read exactly once per call: non-temporal loads stream them past the
// caches instead of allocating lines that will never be hit again.
__device__ __forceinline__ uint4 load_piece(const char* base, uint32_t off) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + off));
  return make_uint4(t[0], t[1], t[2], t[3]);
}

// K of one step: load slot i of lane (kg, r) is position 4*i + kg, piece r, so
// a quarter-wave reads one whole 256-byte (position, head) row.
template <bool TAIL>
__device__ __forceinline__ void issue_k_loads(uint4 (&kreg)[8], const char* base, int kg,
                                              int last, uint32_t row_bytes,
                                              uint32_t lane_bytes) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    kreg[i] = load_piece(base, slot_offset<TAIL>(4 * i + kg, last, row_bytes, lane_bytes));
}

// V of one step: load slot j of lane (kg, r) is the position that reduction
// slot j of k-group kg stands for in the P^T operand: 4*kg + j from the first
// S^T tile, 16 + 4*kg + (j - 4) from the second.
template <bool TAIL>
__device__ __forceinline__ void issue_v_loads(uint4 (&vreg)[8], const char* base, int kg,
                                              int last, uint32_t row_bytes,
                                              uint32_t lane_bytes) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int x = (j < 4) ? (4 * kg + j) : (16 + 4 * kg + (j - 4));
    vreg[j] = load_piece(base, slot_offset<TAIL>(x, last, row_bytes, lane_bytes));
  }
}

// grid.x = batch * max_chunks, grid.y = num_kv_heads / NW, block = NW * 64.
template <int NW>
__global__ __launch_bounds__(NW * 64) void paged_decode_splitk_kernel(
    const uint4* __restrict__ q,          // [B, Hq, 16] pieces
    const char* __restrict__ k_cache,     // [NB, bs, Hkv, 128] bf16
    const char* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables,  // [B, MB]
    const int32_t* __restrict__ context_lens,  // [B]
    uint4* __restrict__ out,              // [B, Hq, 16] pieces (bf16)
    float* __restrict__ part_o,           // [B, max_chunks, Hq, 128]
    float* __restrict__ part_ml,          // [B, max_chunks, Hq, 2]
    int num_heads, int num_kv_heads, int group, int block_size, int max_blocks,
    int num_blocks, int chunk, int max_chunks, float scale_log2e) {
  __shared__ uint4 k_tile[NW][kStep * kLdsRowPieces];

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int r = lane & 15;   // MFMA row/column index inside a 16-wide tile
  const int kg = lane >> 4;  // MFMA k-group (which 8 of the 32 reduction slots)

  const int b = blockIdx.x / max_chunks;
  const int c = blockIdx.x - b * max_chunks;
  // A length beyond what the block table can describe is clamped to it.
  const int ctx = min(context_lens[b], max_blocks * block_size);
  const int t0 = c * chunk;
  if (t0 >= ctx) return;  // also every chunk of an empty sequence
  const int t1 = min(ctx, t0 + chunk);
  const int kvh = blockIdx.y * NW + wave;
  const int nsteps = (t1 - t0 + kStep - 1) / kStep;

  // Q^T as MFMA B operand for the 4 reduction steps over head_dim:
  // lane (column r = query head of the group, k-group kg) holds dims
  // 32*s + 8*kg .. +8.  Columns >= group are zero.
  bf16x8 qreg[4];
  {
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const uint4* qrow = q + ((int64_t)b * num_heads + (int64_t)kvh * group + r) * kRowPieces;
#pragma unroll
    for (int s = 0; s < 4; ++s) qreg[s] = as_bf16x8(r < group ? qrow[4 * s + kg] : zero);
  }

  const uint32_t row_bytes = (uint32_t)num_kv_heads * (kHeadDim * 2);  // one position, all heads
  const uint32_t lane_bytes = (uint32_t)r * 16u;
  const int64_t head_bytes = (int64_t)kvh * (kHeadDim * 2);
  const int32_t* table = block_tables + (int64_t)b * max_blocks;
  uint4* lds = k_tile[wave];

  // wave-uniform byte offset of the first position of a step inside the cache
  auto step_base = [&](int step) -> int64_t {
    const int ts = t0 + step * kStep;
    const int page = ts / block_size;
    const int phys = min(max(table[page], 0), num_blocks - 1);
    return ((int64_t)phys * block_size + (ts - page * block_size)) * row_bytes + head_bytes;
  };

  uint4 kreg[8], vreg[8];
  {
    const int64_t off = step_base(0);
    const int last = min(kStep, t1 - t0) - 1;
    issue_k_loads<true>(kreg, k_cache + off, kg, last, row_bytes, lane_bytes);
    issue_v_loads<true>(vreg, v_cache + off, kg, last, row_bytes, lane_bytes);
  }

  f32x4 acc[8];
#pragma unroll
  for (int jd = 0; jd < 8; ++jd) acc[jd] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = kNegBig;  // running max of raw scores (q.k, unscaled) of column r
  float l_run = 0.f;      // this lane's share of the running sum

  for (int step = 0; step < nsteps; ++step) {
    const int nvalid = min(kStep, t1 - (t0 + step * kStep));
    const bool more = step + 1 < nsteps;
    int64_t next_off = 0;
    int next_last = kStep - 1;
    if (more) {
      next_off = step_base(step + 1);
      next_last = min(kStep, t1 - (t0 + (step + 1) * kStep)) - 1;
    }

    // ---- K: registers -> LDS (row = position, padded), then next K loads ----
#pragma unroll
    for (int i = 0; i < 8; ++i) lds[(4 * i + kg) * kLdsRowPieces + r] = kreg[i];
    if (more) {
      if (next_last == kStep - 1)
        issue_k_loads<false>(kreg, k_cache + next_off, kg, next_last, row_bytes, lane_bytes);
      else
        issue_k_loads<true>(kreg, k_cache + next_off, kg, next_last, row_bytes, lane_bytes);
    }

    // ---- S^T = K . Q^T for two 16-position tiles ----
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bf16x8 a0 = as_bf16x8(lds[r * kLdsRowPieces + 4 * s + kg]);
      const bf16x8 a1 = as_bf16x8(lds[(16 + r) * kLdsRowPieces + 4 * s + kg]);
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qreg[s], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qreg[s], s1, 0, 0, 0);
    }

    // ---- online softmax; lane holds positions 4*kg+e (s0) and 16+4*kg+e (s1) ----
    if (nvalid < kStep) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (4 * kg + e >= nvalid) s0[e] = kNegBig;
        if (16 + 4 * kg + e >= nvalid) s1[e] = kNegBig;
      }
    }
    float mx = fmaxf(fmaxf(fmaxf(s0[0], s0[1]), fmaxf(s0[2], s0[3])),
                     fmaxf(fmaxf(s1[0], s1[1]), fmaxf(s1[2], s1[3])));
    mx = wave_xor_max(mx, 16);
    mx = wave_xor_max(mx, 32);
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2e);
    const float mneg = -m_new * scale_log2e;
    m_run = m_new;
    float p0[4], p1[4];
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      p0[e] = __builtin_amdgcn_exp2f(fmaf(s0[e], scale_log2e, mneg));
      p1[e] = __builtin_amdgcn_exp2f(fmaf(s1[e], scale_log2e, mneg));
      psum += p0[e] + p1[e];
    }
    l_run = fmaf(l_run, alpha, psum);
    uint4 pbits;
    pbits.x = pack_bf16x2(p0[0], p0[1]);
    pbits.y = pack_bf16x2(p0[2], p0[3]);
    pbits.z = pack_bf16x2(p1[0], p1[1]);
    pbits.w = pack_bf16x2(p1[2], p1[3]);
    const bf16x8 pb = as_bf16x8(pbits);

    // ---- V: in-lane 8x8 transpose (positions x dims), then next V loads ----
    uint4 vt[8];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t vw[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        vw[j] = w == 0 ? vreg[j].x : w == 1 ? vreg[j].y : w == 2 ? vreg[j].z : vreg[j].w;
      // even dim of the pair: low halves; odd dim: high halves
      vt[2 * w].x = __builtin_amdgcn_perm(vw[1], vw[0], 0x05040100u);
      vt[2 * w].y = __builtin_amdgcn_perm(vw[3], vw[2], 0x05040100u);
      vt[2 * w].z = __builtin_amdgcn_perm(vw[5], vw[4], 0x05040100u);
      vt[2 * w].w = __builtin_amdgcn_perm(vw[7], vw[6], 0x05040100u);
      vt[2 * w + 1].x = __builtin_amdgcn_perm(vw[1], vw[0], 0x07060302u);
      vt[2 * w + 1].y = __builtin_amdgcn_perm(vw[3], vw[2], 0x07060302u);
      vt[2 * w + 1].z = __builtin_amdgcn_perm(vw[5], vw[4], 0x07060302u);
      vt[2 * w + 1].w = __builtin_amdgcn_perm(vw[7], vw[6], 0x07060302u);
    }
    if (more) {
      if (next_last == kStep - 1)
        issue_v_loads<false>(vreg, v_cache + next_off, kg, next_last, row_bytes, lane_bytes);
      else
        issue_v_loads<true>(vreg, v_cache + next_off, kg, next_last, row_bytes, lane_bytes);
    }

    // ---- O^T = alpha * O^T + V^T . P^T ----
#pragma unroll
    for (int jd = 0; jd < 8; ++jd) {
      acc[jd] *= alpha;
      acc[jd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vt[jd]), pb, acc[jd], 0, 0, 0);
    }
  }

  // total of the running sum over the 4 k-groups that share column r
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);

  if (r >= group) return;
  const int head = kvh * group + r;
  // acc[jd][e] is O[head][dim = 32*kg + 8*e + jd]
  const int nchunks = (ctx + chunk - 1) / chunk;
  if (nchunks == 1) {
    const float inv = 1.0f / (l_run + 1e-9f);
    uint4* orow = out + ((int64_t)b * num_heads + head) * kRowPieces + 4 * kg;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      uint4 o;
      o.x = pack_bf16x2(acc[0][e] * inv, acc[1][e] * inv);
      o.y = pack_bf16x2(acc[2][e] * inv, acc[3][e] * inv);
      o.z = pack_bf16x2(acc[4][e] * inv, acc[5][e] * inv);
      o.w = pack_bf16x2(acc[6][e] * inv, acc[7][e] * inv);
      orow[e] = o;
    }
  } else {
    const int64_t slot = ((int64_t)b * max_chunks + c) * num_heads + head;
    float4* prow = reinterpret_cast<float4*>(part_o + slot * kHeadDim + 32 * kg);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      prow[2 * e] = make_float4(acc[0][e], acc[1][e], acc[2][e], acc[3][e]);
      prow[2 * e + 1] = make_float4(acc[4][e], acc[5][e], acc[6][e], acc[7][e]);
    }
    if (kg == 0) {
      reinterpret_cast<float2*>(part_ml)[slot] = make_float2(m_run, l_run);
    }
  }
}

// Merge the per-chunk partials of one (sequence, query head).  grid = (B, Hq),
// block = 128 lanes, one per output dim.
__global__ __launch_bounds__(kHeadDim) void paged_decode_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const int32_t* __restrict__ context_lens, uint16_t* __restrict__ out, int num_heads,
    int chunk, int max_chunks, int max_positions, float scale_log2e) {
  const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
  const int ctx = min(context_lens[b], max_positions);
  const int nchunks = ctx <= 0 ? 0 : (ctx + chunk - 1) / chunk;
  if (nchunks == 1) return;  // written by the split-K kernel itself
  uint16_t* o = out + ((int64_t)b * num_heads + h) * kHeadDim + d;
  if (nchunks == 0) {  // empty sequence: 0 / (0 + 1e-9)
    *o = 0;
    return;
  }
  const int64_t base = (int64_t)b * max_chunks * num_heads + h;
  const float2* ml = reinterpret_cast<const float2*>(part_ml);
  float m = kNegBig;
  for (int c = 0; c < nchunks; ++c) m = fmaxf(m, ml[base + (int64_t)c * num_heads].x);
  float num = 0.f, den = 0.f;
  for (int c = 0; c < nchunks; ++c) {
    const int64_t slot = base + (int64_t)c * num_heads;
    const float2 v = ml[slot];
    const float w = __builtin_amdgcn_exp2f((v.x - m) * scale_log2e);
    den = fmaf(w, v.y, den);
    num = fmaf(w, part_o[slot * kHeadDim + d], num);
  }
  const float res = num / (den + 1e-9f);
  *o = (uint16_t)(pack_bf16x2(res, 0.f) & 0xFFFFu);
}

int round_up(int x, int m) { return (x + m - 1) / m * m; }

}  // namespace

extern "C" int32_t nvj_paged_decode_default_chunk(int32_t batch, int32_t num_kv_heads,
                                                  int32_t max_blocks, int32_t block_size) {
  if (batch <= 0 || num_kv_heads <= 0 || max_blocks <= 0 || block_size <= 0) return 256;
  // One workgroup (8 waves at ~230 VGPRs) is resident per CU, and the kernel
  // is fastest when a launch is exactly one workgroup per CU (256 on MI355X):
  // pick the chunk that gives that when every sequence is at full length, if
  // it is at most 2048 positions.  Beyond that the launch runs in several
  // rounds anyway and 1024 keeps ragged batches balanced (a long chunk that
  // starts late becomes the tail of the whole launch).  Below 128 positions
  // the partials only add combine work.
  const int64_t positions = (int64_t)batch * max_blocks * block_size;
  int64_t chunk = (positions + 255) / 256;
  if (chunk < 128) chunk = 128;
  if (chunk > 2048) chunk = 1024;
  return round_up((int)chunk, kStep);
}

static int resolve_chunk(int32_t batch, int32_t num_kv_heads, int32_t max_blocks,
                         int32_t block_size, int32_t chunk) {
  if (chunk == 0) chunk = nvj_paged_decode_default_chunk(batch, num_kv_heads, max_blocks, block_size);
  return chunk;
}

extern "C" size_t nvj_paged_decode_workspace_bytes(int32_t batch, int32_t num_heads,
                                                   int32_t head_dim, int32_t max_blocks,
                                                   int32_t block_size, int32_t num_kv_heads,
                                                   int32_t chunk) {
  if (batch <= 0 || num_heads <= 0 || head_dim <= 0 || max_blocks <= 0 || block_size <= 0 ||
      chunk < 0 || chunk % kStep != 0)
    return 0;
  chunk = resolve_chunk(batch, num_kv_heads, max_blocks, block_size, chunk);
  const int64_t max_chunks = ((int64_t)max_blocks * block_size + chunk - 1) / chunk;
  const int64_t slots = (int64_t)batch * max_chunks * num_heads;
  return (size_t)(slots * (head_dim + 2) * sizeof(float));
}

extern "C" int nvj_paged_decode_launch_phases(void* stream, const void* q, const void* k_cache,
                                              const void* v_cache, const int32_t* block_tables,
                                              const int32_t* context_lens, void* out,
                                              void* workspace, size_t workspace_bytes,
                                              int32_t batch, int32_t num_heads,
                                              int32_t num_kv_heads, int32_t head_dim,
                                              int32_t block_size, int32_t max_blocks,
                                              int32_t num_blocks, float scale, int32_t chunk,
                                              uint32_t phases) {
  if (batch < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 ||
      max_blocks < 0 || num_blocks <= 0 || chunk < 0)
    return NVJ_ERR_BAD_SHAPE;
  if (num_heads % num_kv_heads != 0) return NVJ_ERR_BAD_SHAPE;
  const int group = num_heads / num_kv_heads;
  if (head_dim != kHeadDim || group > 16 || block_size % kStep != 0 || chunk % kStep != 0)
    return NVJ_ERR_UNSUPPORTED;
  if (batch == 0) return NVJ_OK;
  if (!q || !k_cache || !v_cache || !context_lens || !out) return NVJ_ERR_NULL_POINTER;
  if (max_blocks > 0 && !block_tables) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_cache) |
       reinterpret_cast<uintptr_t>(v_cache) | reinterpret_cast<uintptr_t>(out) |
       reinterpret_cast<uintptr_t>(workspace)) & 15u)
    return NVJ_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float scale_log2e = scale * kLog2e;

  int max_chunks = 1;
  float* part_o = nullptr;
  float* part_ml = nullptr;
  if (max_blocks > 0) {
    chunk = resolve_chunk(batch, num_kv_heads, max_blocks, block_size, chunk);
    const int64_t mc = ((int64_t)max_blocks * block_size + chunk - 1) / chunk;
    const int64_t slots = (int64_t)batch * mc * num_heads;
    if ((int64_t)batch * mc > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
    const size_t need = (size_t)slots * (kHeadDim + 2) * sizeof(float);
    if (!workspace || workspace_bytes < need) return NVJ_ERR_WORKSPACE;
    max_chunks = (int)mc;
    part_o = static_cast<float*>(workspace);
    part_ml = part_o + slots * kHeadDim;

    const int nw = num_kv_heads % 8 == 0 ? 8 : num_kv_heads % 4 == 0 ? 4 : num_kv_heads % 2 == 0 ? 2 : 1;
    dim3 grid((unsigned)(batch * max_chunks), (unsigned)(num_kv_heads / nw));
    const uint4* q4 = static_cast<const uint4*>(q);
    const char* k4 = static_cast<const char*>(k_cache);
    const char* v4 = static_cast<const char*>(v_cache);
    uint4* o4 = static_cast<uint4*>(out);
    if (phases & NVJ_PHASE_SPLITK) {
#define NVJ_LAUNCH_SPLITK(NWV)                                                               \
  paged_decode_splitk_kernel<NWV><<<grid, dim3(NWV * 64), 0, s>>>(                           \
      q4, k4, v4, block_tables, context_lens, o4, part_o, part_ml, num_heads, num_kv_heads,  \
      group, block_size, max_blocks, num_blocks, chunk, max_chunks, scale_log2e)
    switch (nw) {
      case 8: NVJ_LAUNCH_SPLITK(8); break;
      case 4: NVJ_LAUNCH_SPLITK(4); break;
      case 2: NVJ_LAUNCH_SPLITK(2); break;
      default: NVJ_LAUNCH_SPLITK(1); break;
    }
#undef NVJ_LAUNCH_SPLITK
      if (hipGetLastError() != hipSuccess) return NVJ_ERR_LAUNCH;
    }
  } else {
    chunk = kStep;  // no pages at all: every sequence is empty, combine writes zeros
  }
  if (!(phases & NVJ_PHASE_COMBINE)) return NVJ_OK;
  paged_decode_combine_kernel<<<dim3((unsigned)batch, (unsigned)num_heads), dim3(kHeadDim), 0, s>>>(
      part_o, part_ml, context_lens, static_cast<uint16_t*>(out), num_heads, chunk, max_chunks,
      max_blocks * block_size, scale_log2e);
  return hipGetLastError() == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

extern "C" int nvj_paged_decode_launch(void* stream, const void* q, const void* k_cache,
                                       const void* v_cache, const int32_t* block_tables,
                                       const int32_t* context_lens, void* out, void* workspace,
                                       size_t workspace_bytes, int32_t batch, int32_t num_heads,
                                       int32_t num_kv_heads, int32_t head_dim,
                                       int32_t block_size, int32_t max_blocks,
                                       int32_t num_blocks, float scale, int32_t chunk) {
  return nvj_paged_decode_launch_phases(stream, q, k_cache, v_cache, block_tables, context_lens,
                                        out, workspace, workspace_bytes, batch, num_heads,
                                        num_kv_heads, head_dim, block_size, max_blocks,
                                        num_blocks, scale, chunk,
                                        NVJ_PHASE_SPLITK | NVJ_PHASE_COMBINE);
}

extern "C" const char* nvj_error_string(int code) {
  switch (code) {
    case NVJ_OK: return "ok";
    case NVJ_ERR_NULL_POINTER: return "a required pointer is NULL";
    case NVJ_ERR_BAD_SHAPE: return "invalid shape or size argument";
    case NVJ_ERR_UNSUPPORTED: return "unsupported head_dim / group size / block size / chunk";
    case NVJ_ERR_WORKSPACE: return "workspace missing, too small or misaligned";
    case NVJ_ERR_LAUNCH: return "kernel launch failed";
    case NVJ_ERR_BAD_DTYPE: return "unknown element type code";
    default: return "unknown error code";
  }
}

extern "C" int nvj_abi_version(void) { return NVJ_ABI_VERSION; }

// Split-K paged decode attention for gfx950 (CDNA4, wave64) and its combine pass.
//
// Stands in for paged_attention -> paged_decode_attention_vectorized
// (layers/pallas_attention.py:465-507, :146-238 of the reference) and for the
// gather + dot_product_attention fallback (layers/attention.py:399-434).
//
// Work split.  A workgroup handles a run of positions for NW KV heads at once,
// one wave per KV head, so the workgroup as a whole streams whole 2 KiB cache
// rows (all heads of a position are contiguous in the [page, position, head,
// dim] layout).  A wave owns the G query heads of its KV head, so every K/V
// byte is fetched once per group.  The runs are either equal cuts of all the
// steps of the batch, derived on the device from context_lens (balanced split,
// the default), or fixed chunks of each sequence.  A third mode finishes every
// sequence inside one workgroup (its waves are a few KV heads x equal parts of
// the sequence, merged through LDS): one launch, no workspace, for batches of
// similar lengths.
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
// In the first two modes the partial (unnormalised O, running max, running
// sum) of every segment goes to the workspace and the combine kernel merges the
// segments of a sequence; a sequence that is one segment is written directly.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "nvj_paged_attn.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kMaxHeadDim = 128;     // head_dim is a template parameter: 128 or 64
constexpr int kStep = 32;            // positions per inner step
// A (position, head) row of D bf16 is D/8 16-byte pieces; the LDS tile pads a
// row by one piece so that the 16 rows an MFMA operand read touches fall on
// different banks.
template <int D> struct HeadDim {
  static_assert(D == 128 || D == 64, "head_dim 128 or 64");
  static constexpr int kPieces = D / 8;             // 16 or 8
  static constexpr int kLdsRowPieces = kPieces + 1;
  static constexpr int kPosPerLoad = 64 / kPieces;  // positions one 64-lane load covers: 4 or 8
  static constexpr int kKLoads = kStep / kPosPerLoad;  // K loads per lane per step: 8 or 4
  static constexpr int kQkSteps = D / 32;           // MFMA reduction steps of Q.K: 4 or 2
};
constexpr float kNegBig = -1.0e30f;  // stands for -inf without inf-inf hazards
constexpr float kLog2e = 1.4426950408889634f;

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

// The cache element type: bf16 (F16 = false) or IEEE half (F16 = true).  The
// kernels move 16-bit patterns; only the matrix instruction, the rounding of
// the probabilities and of the output depend on the type.
template <bool F16> struct Elem;
template <> struct Elem<false> {
  static __device__ __forceinline__ f32x4 mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    bf16x2 p = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, p);
  }
};
template <> struct Elem<true> {
  static __device__ __forceinline__ f32x4 mfma(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
    f16x2 p = {(_Float16)lo, (_Float16)hi};   // round to nearest even
    return __builtin_bit_cast(uint32_t, p);
  }
};


__device__ __forceinline__ float wave_xor_max(float x, int mask) {
  return fmaxf(x, __shfl_xor(x, mask, 64));
}

// K/V are read exactly once per call: non-temporal loads stream them past the
// caches instead of allocating lines that will never be hit again.  `base` is
// wave-uniform (scalar registers), `off` the lane's 32-bit byte offset: a step
// never leaves its page, so offsets stay below block_size * row_bytes.
__device__ __forceinline__ uint4 load_piece(const char* base, uint32_t off) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + off));
  return make_uint4(t[0], t[1], t[2], t[3]);
}

// K of one step: 64 lanes cover kPosPerLoad whole (position, head) rows per
// load (lane -> position lane / kPieces, piece lane % kPieces), so every group
// of kPieces lanes reads one contiguous row (a quarter-wave at head_dim 128).
// In a full step the position splits into a uniform part (folded into the
// scalar base) and one per-lane offset shared by all loads; a TAIL step clamps
// every slot to the last live position so that nothing at or beyond the
// context length is ever read.
template <bool TAIL, int D>
__device__ __forceinline__ void issue_k_loads(uint4 (&kreg)[HeadDim<D>::kKLoads],
                                              const char* base, int lane, int last,
                                              uint32_t row_bytes) {
  using H = HeadDim<D>;
  const int pos_lane = lane / H::kPieces;
  const uint32_t piece_bytes = (uint32_t)(lane % H::kPieces) * 16u;
#pragma unroll
  for (int i = 0; i < H::kKLoads; ++i) {
    if constexpr (TAIL) {
      kreg[i] = load_piece(
          base, (uint32_t)min(H::kPosPerLoad * i + pos_lane, last) * row_bytes + piece_bytes);
    } else {
      kreg[i] = load_piece(base + (size_t)(H::kPosPerLoad * i) * row_bytes,
                           (uint32_t)pos_lane * row_bytes + piece_bytes);
    }
  }
}

// V of one step: load slot j of lane (kg, r) is the position that reduction
// slot j of k-group kg stands for in the P^T operand: 4*kg + j from the first
// S^T tile, 16 + 4*kg + (j - 4) from the second.
template <bool TAIL, int D>
__device__ __forceinline__ void issue_v_loads(uint4 (&vreg)[8], const char* base, int kg, int r,
                                              int last, uint32_t row_bytes) {
  // lane (kg, r) fetches piece r (dims 8r .. 8r+7) of its 8 positions; at
  // head_dim 64 there are only 8 pieces and lanes r >= 8 hold zeros
  const bool live = r < HeadDim<D>::kPieces;
  const uint32_t lane_bytes = (uint32_t)r * 16u;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int uni = (j < 4) ? j : (16 + j - 4);   // uniform part of the position
    if (!live) {
      vreg[j] = zero;
    } else if constexpr (TAIL) {
      vreg[j] = load_piece(base, (uint32_t)min(4 * kg + uni, last) * row_bytes + lane_bytes);
    } else {
      vreg[j] = load_piece(base + (size_t)uni * row_bytes,
                           (uint32_t)(4 * kg) * row_bytes + lane_bytes);
    }
  }
}

// Read-only int32 metadata (block tables, context lengths) is never written
// while a launch runs.  Reading it through the constant address space tells
// the compiler so: a wave-uniform index then becomes a scalar load (s_load)
// even after the kernel has issued stores of its own, instead of a vector load
// whose result has to be moved back to the scalar unit.
typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;
__device__ __forceinline__ const_i32_ptr as_constant(const int32_t* p) {
  return (const_i32_ptr)(uintptr_t)p;
}

// Everything shared by the launch: pointers and problem shape.
struct DecodeArgs {
  const uint4* q;              // [B, Hq, 16] pieces
  const char* k_cache;         // [NB, bs, Hkv, 128] bf16
  const char* v_cache;
  const int32_t* block_tables; // [B, MB]
  const int32_t* context_lens; // [B]
  uint4* out;                  // [B, Hq, 16] pieces (bf16)
  float* part_o;               // [slots, Hq, 128]
  float* part_ml;              // [slots, Hq, 2]
  // num_kv_heads and group describe the heads as the kernels walk them: with
  // more than 16 query heads per cache head, a cache head is walked as kv_rep
  // "virtual" KV heads of group = G / kv_rep query heads each (kv_rep = 1
  // otherwise); cache_kv_heads is the number of heads a cache row really holds.
  int num_heads, num_kv_heads, group, kv_rep, cache_kv_heads, block_size, max_blocks, num_blocks;
  float scale_log2e;
};

// One wave's share of one segment: positions [t0, t1) of sequence b for KV head
// kvh; t0 is a multiple of 32, t0 < t1.  Leaves the unnormalised result in
// registers: acc[jd][e] is O[head kvh*group + r][dim 32*kg + 8*e + jd] for the
// lane (r = lane & 15, kg = lane >> 4), m_run the maximum raw score and l_run
// the sum of exp((score - m_run) * scale) of that head (the same in the four
// lanes that share r).  Lanes with r >= group hold padding.
template <int D, bool F16>
__device__ __forceinline__ void compute_segment(const DecodeArgs& a, uint4* lds, int b, int kvh,
                                                int t0, int t1, int lane, f32x4 (&acc)[8],
                                                float& m_run, float& l_run) {
  using H = HeadDim<D>;
  const int r = lane & 15;   // MFMA row/column index inside a 16-wide tile
  const int kg = lane >> 4;  // MFMA k-group (which 8 of the 32 reduction slots)
  const uint4* __restrict__ q = a.q;
  const char* __restrict__ k_cache = a.k_cache;
  const char* __restrict__ v_cache = a.v_cache;
  const int num_heads = a.num_heads, group = a.group, block_size = a.block_size;
  const int num_blocks = a.num_blocks;
  const float scale_log2e = a.scale_log2e;
  const int nsteps = (t1 - t0 + kStep - 1) / kStep;

  // Q^T as MFMA B operand for the D/32 reduction steps over head_dim:
  // lane (column r = query head of the group, k-group kg) holds dims
  // 32*s + 8*kg .. +8.  Columns >= group are zero.
  uint4 qreg[H::kQkSteps];
  {
    // lanes of padding columns read the group's last head (always in range)
    // and then drop it, so the loads stay unconditional 16-byte loads
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const uint4* qrow =
        q + ((int64_t)b * num_heads + (int64_t)kvh * group + min(r, group - 1)) * H::kPieces;
#pragma unroll
    for (int s = 0; s < H::kQkSteps; ++s) {
      const uint4 v = qrow[4 * s + kg];
      qreg[s] = r < group ? v : zero;
    }
  }

  const uint32_t row_bytes = (uint32_t)a.cache_kv_heads * (D * 2);  // one position, all heads
  const int64_t head_bytes = (int64_t)(kvh / a.kv_rep) * (D * 2);
  const const_i32_ptr table = as_constant(a.block_tables + (int64_t)b * a.max_blocks);

  // wave-uniform byte offset of the first position of a step inside the cache
  auto step_base = [&](int step) -> int64_t {
    const int ts = t0 + step * kStep;
    const int page = ts / block_size;
    const int phys = min(max(table[page], 0), num_blocks - 1);
    return ((int64_t)phys * block_size + (ts - page * block_size)) * row_bytes + head_bytes;
  };

  uint4 kreg[H::kKLoads], vreg[8];
  {
    const int64_t off = step_base(0);
    const int last = min(kStep, t1 - t0) - 1;
    issue_k_loads<true, D>(kreg, k_cache + off, lane, last, row_bytes);
    issue_v_loads<true, D>(vreg, v_cache + off, kg, r, last, row_bytes);
  }

#pragma unroll
  for (int jd = 0; jd < 8; ++jd) acc[jd] = f32x4{0.f, 0.f, 0.f, 0.f};
  m_run = kNegBig;  // running max of raw scores (q.k, unscaled) of column r
  l_run = 0.f;      // this lane's share of the running sum

  // the page lookup of a step is started two steps ahead, so that its latency
  // is not in front of the loads that need the address
  int64_t off_ahead = nsteps > 1 ? step_base(1) : 0;
  for (int step = 0; step < nsteps; ++step) {
    const int nvalid = min(kStep, t1 - (t0 + step * kStep));
    const bool more = step + 1 < nsteps;
    const int64_t next_off = off_ahead;
    int next_last = kStep - 1;
    if (more) next_last = min(kStep, t1 - (t0 + (step + 1) * kStep)) - 1;
    if (step + 2 < nsteps) off_ahead = step_base(step + 2);

    // ---- K: registers -> LDS (row = position, padded), then next K loads ----
#pragma unroll
    for (int i = 0; i < H::kKLoads; ++i)
      lds[(H::kPosPerLoad * i + lane / H::kPieces) * H::kLdsRowPieces + lane % H::kPieces] =
          kreg[i];
    if (more) {
      if (next_last == kStep - 1)
        issue_k_loads<false, D>(kreg, k_cache + next_off, lane, next_last, row_bytes);
      else
        issue_k_loads<true, D>(kreg, k_cache + next_off, lane, next_last, row_bytes);
    }

    // ---- S^T = K . Q^T for two 16-position tiles ----
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < H::kQkSteps; ++s) {
      const uint4 a0 = lds[r * H::kLdsRowPieces + 4 * s + kg];
      const uint4 a1 = lds[(16 + r) * H::kLdsRowPieces + 4 * s + kg];
      s0 = Elem<F16>::mfma(a0, qreg[s], s0);
      s1 = Elem<F16>::mfma(a1, qreg[s], s1);
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
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      p0[e] = __builtin_amdgcn_exp2f(fmaf(s0[e], scale_log2e, mneg));
      p1[e] = __builtin_amdgcn_exp2f(fmaf(s1[e], scale_log2e, mneg));
    }
    if (nvalid < kStep) {
      // positions past the end weigh exactly 0 whatever the scale (at scale 0
      // the exponential of a masked score is 1, not 0)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (4 * kg + e >= nvalid) p0[e] = 0.f;
        if (16 + 4 * kg + e >= nvalid) p1[e] = 0.f;
      }
    }
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) psum += p0[e] + p1[e];
    l_run = fmaf(l_run, alpha, psum);
    uint4 pbits;
    pbits.x = Elem<F16>::pack2(p0[0], p0[1]);
    pbits.y = Elem<F16>::pack2(p0[2], p0[3]);
    pbits.z = Elem<F16>::pack2(p1[0], p1[1]);
    pbits.w = Elem<F16>::pack2(p1[2], p1[3]);

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
        issue_v_loads<false, D>(vreg, v_cache + next_off, kg, r, next_last, row_bytes);
      else
        issue_v_loads<true, D>(vreg, v_cache + next_off, kg, r, next_last, row_bytes);
    }

    // ---- O^T = alpha * O^T + V^T . P^T ----
#pragma unroll
    for (int jd = 0; jd < 8; ++jd) {
      acc[jd] *= alpha;
      acc[jd] = Elem<F16>::mfma(vt[jd], pbits, acc[jd]);
    }
  }

  // total of the running sum over the 4 k-groups that share column r
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
}

// ---------------------------------------------------------------------------
// Measurement variant: the same segment with both products on the vector ALU
// (v_dot2c_f32_bf16) instead of the matrix cores, so that the choice between
// the two can be timed rather than argued.  head_dim 128, bf16, exactly G = 2,
// 4 or 8 query heads per KV head.  Same loads, same page walk, same results
// layout as compute_segment; only the arithmetic between them differs:
//   * Q.K: lane (pl = lane / 16, pc = lane % 16) holds dims 8*pc .. +8 of
//     position 4*i + pl for its 8 K loads i and the same dims of all G query
//     rows, so 4 dot2 give a 1/16 partial of score (i, h).  The 8*G partials
//     per lane are summed over the 16 lanes of a row by a halving exchange
//     (DPP mirror, half mirror, two quad permutes): each step a lane keeps
//     one half of its values and adds the partner's copy of that half, which
//     leaves lane pc with the 8*G/16 complete scores of one head.
//   * softmax on those few scores per lane; the probabilities (bf16) and the
//     rescale factors travel to the P.V layout through the wave's LDS tile.
//   * P.V: lane (kg, r) holds 8 positions x 8 dims of V, transposed in-lane
//     into (position pair) x dim words as in the MFMA path, then 4 dot2 per
//     (head, dim) against the matching probability pairs; the four position
//     groups kg are summed once at the end.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a),
                                         __builtin_bit_cast(bf16x2, b), c, false);
}

// value of the lane that DPP control CTRL pairs this lane with (same row of 16)
template <int CTRL> __device__ __forceinline__ float dpp_partner(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}

// One halving step over v[0 .. 2*HALF): the lane whose `upper` is false keeps
// the even entries, its partner (upper true) the odd ones; each adds the
// partner's copy of what it keeps.  Result in v[0 .. HALF).
template <int CTRL, int HALF, int N>
__device__ __forceinline__ void halve_across(float (&v)[N], bool upper) {
#pragma unroll
  for (int j = 0; j < HALF; ++j) {
    const float keep = upper ? v[2 * j + 1] : v[2 * j];
    const float send = upper ? v[2 * j] : v[2 * j + 1];
    v[j] = keep + dpp_partner<CTRL>(send);
  }
}

constexpr int kDppQuadXor1 = 0xB1;      // quad_perm [1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;      // quad_perm [2,3,0,1]
constexpr int kDppRowMirror = 0x140;    // lane i <-> 15 - i
constexpr int kDppHalfMirror = 0x141;   // lane i <-> i ^ 7

template <int G>
__device__ __forceinline__ void compute_segment_valu(const DecodeArgs& a, uint4* lds, int b,
                                                     int kvh, int t0, int t1, int lane,
                                                     f32x4 (&acc_out)[8], float& m_out,
                                                     float& l_out) {
  static_assert(G == 2 || G == 4 || G == 8, "vector-ALU variant: 2, 4 or 8 query heads");
  constexpr int D = 128;
  using H = HeadDim<D>;
  // the 8 K loads of a step are scored in batches of LB loads = NB partial
  // scores per lane, which the exchange turns into NB / 16 complete ones
  constexpr int LB = G <= 4 ? 8 : 32 / G;   // K loads per batch
  constexpr int NB = LB * G;                // partial scores per lane and batch (16 or 32)
  constexpr int CB = NB / 16;               // complete scores per lane and batch
  constexpr int NS = 8 / LB * CB;           // complete scores per lane and step
  const int r = lane & 15, kg = lane >> 4;   // (piece, position group) in either layout
  const char* __restrict__ k_cache = a.k_cache;
  const char* __restrict__ v_cache = a.v_cache;
  const int block_size = a.block_size, num_blocks = a.num_blocks;
  const float scale_log2e = a.scale_log2e;
  const int nsteps = (t1 - t0 + kStep - 1) / kStep;

  // wave-private LDS: probabilities [G][32] bf16, rescale factors [G] f32,
  // and at the end of the segment the results [G][128] f32 + (max, sum) [G][2]
  uint16_t* lds_p = reinterpret_cast<uint16_t*>(lds);
  float* lds_alpha = reinterpret_cast<float*>(lds) + 256;   // byte 1024
  float* lds_o = reinterpret_cast<float*>(lds) + 512;       // byte 2048
  float* lds_ml = lds_o + G * D;
  static_assert((512 + 8 * 128 + 16) * 4 <= kStep * H::kLdsRowPieces * 16, "fits the K tile");

  // dims 8*r .. +8 of every query row of the group: in registers up to 4 rows,
  // in the wave's LDS tile beyond (read back per batch, the same address in
  // the four lanes that share r), which keeps the 8-row form free of spills
  constexpr bool kQInLds = G > 4;
  uint4* lds_q = lds + 400;   // byte 6400, behind the hand-over area; G * 16 pieces
  static_assert(400 + 8 * 16 <= kStep * H::kLdsRowPieces, "q pieces fit the K tile");
  uint4 qv[kQInLds ? 1 : G];
  if constexpr (kQInLds) {
#pragma unroll
    for (int h = kg; h < G; h += 4)
      lds_q[h * H::kPieces + r] =
          a.q[((int64_t)b * a.num_heads + (int64_t)kvh * G + h) * H::kPieces + r];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  } else {
#pragma unroll
    for (int h = 0; h < G; ++h)
      qv[h] = a.q[((int64_t)b * a.num_heads + (int64_t)kvh * G + h) * H::kPieces + r];
  }

  // the scores this lane owns after the exchange: entry c of a batch is partial
  // index n = low + 16 * c, low = the bits of r in reverse order; n = h + G * i
  // with i the load inside the batch
  const int low = ((r >> 3) & 1) | ((r >> 1) & 2) | ((r << 1) & 4) | ((r << 3) & 8);
  const int my_h = low % G;
  int my_pos[NS];   // position inside the step, entry = batch * CB + c
#pragma unroll
  for (int bt = 0; bt < 8 / LB; ++bt)
#pragma unroll
    for (int c = 0; c < CB; ++c) my_pos[bt * CB + c] = 4 * (bt * LB + (low + 16 * c) / G) + kg;
  // one lane per head publishes that head's values: the first of those that share it
  const bool publisher = kg == 0 && (r & (16 / G - 1)) == 0;

  const uint32_t row_bytes = (uint32_t)a.cache_kv_heads * (D * 2);
  const int64_t head_bytes = (int64_t)(kvh / a.kv_rep) * (D * 2);
  const const_i32_ptr table = as_constant(a.block_tables + (int64_t)b * a.max_blocks);
  auto step_base = [&](int step) -> int64_t {
    const int ts = t0 + step * kStep;
    const int page = ts / block_size;
    const int phys = min(max(table[page], 0), num_blocks - 1);
    return ((int64_t)phys * block_size + (ts - page * block_size)) * row_bytes + head_bytes;
  };

  uint4 kreg[H::kKLoads], vreg[8];
  {
    const int64_t off = step_base(0);
    const int last = min(kStep, t1 - t0) - 1;
    issue_k_loads<true, D>(kreg, k_cache + off, lane, last, row_bytes);
    issue_v_loads<true, D>(vreg, v_cache + off, kg, r, last, row_bytes);
  }

  float acc[G][8];   // O[head h][dim 8*r + jd], this lane's position group only
#pragma unroll
  for (int h = 0; h < G; ++h)
#pragma unroll
    for (int jd = 0; jd < 8; ++jd) acc[h][jd] = 0.f;
  float m_run = kNegBig, l_run = 0.f;   // of head my_h; l_run is this lane's share

  // the page lookup of a step is started two steps ahead, so that its latency
  // is not in front of the loads that need the address
  int64_t off_ahead = nsteps > 1 ? step_base(1) : 0;
  for (int step = 0; step < nsteps; ++step) {
    const int nvalid = min(kStep, t1 - (t0 + step * kStep));
    const bool more = step + 1 < nsteps;
    const int64_t next_off = off_ahead;
    int next_last = kStep - 1;
    if (more) next_last = min(kStep, t1 - (t0 + (step + 1) * kStep)) - 1;
    if (step + 2 < nsteps) off_ahead = step_base(step + 2);

    // ---- scores, batch by batch, then next K loads ----
    float v[NS];
#pragma unroll
    for (int bt = 0; bt < 8 / LB; ++bt) {
      float part[NB];
#pragma unroll
      for (int i = 0; i < LB; ++i)
#pragma unroll
        for (int h = 0; h < G; ++h) {
          const uint4 kk = kreg[bt * LB + i];
          const uint4 qq = kQInLds ? lds_q[h * H::kPieces + r] : qv[kQInLds ? 0 : h];
          float s = dot2_bf16(kk.x, qq.x, 0.f);
          s = dot2_bf16(kk.y, qq.y, s);
          s = dot2_bf16(kk.z, qq.z, s);
          part[h + G * i] = dot2_bf16(kk.w, qq.w, s);
        }
      halve_across<kDppRowMirror, NB / 2>(part, (r & 8) != 0);
      halve_across<kDppHalfMirror, NB / 4>(part, (r & 4) != 0);
      halve_across<kDppQuadXor2, NB / 8>(part, (r & 2) != 0);
      halve_across<kDppQuadXor1, NB / 16>(part, (r & 1) != 0);
#pragma unroll
      for (int c = 0; c < CB; ++c) v[bt * CB + c] = part[c];
    }
    if (more) {
      if (next_last == kStep - 1)
        issue_k_loads<false, D>(kreg, k_cache + next_off, lane, next_last, row_bytes);
      else
        issue_k_loads<true, D>(kreg, k_cache + next_off, lane, next_last, row_bytes);
    }

    // ---- online softmax of head my_h over the lanes that share it ----
    float mx = kNegBig;
#pragma unroll
    for (int c = 0; c < NS; ++c) {
      if (my_pos[c] >= nvalid) v[c] = kNegBig;
      mx = fmaxf(mx, v[c]);
    }
    mx = fmaxf(mx, dpp_partner<kDppQuadXor1>(mx));
    if (G <= 4) mx = fmaxf(mx, dpp_partner<kDppQuadXor2>(mx));
    if (G <= 2) mx = fmaxf(mx, dpp_partner<kDppHalfMirror>(mx));
    mx = wave_xor_max(mx, 16);
    mx = wave_xor_max(mx, 32);
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2e);
    const float mneg = -m_new * scale_log2e;
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int c = 0; c < NS; ++c) {
      float p = __builtin_amdgcn_exp2f(fmaf(v[c], scale_log2e, mneg));
      if (my_pos[c] >= nvalid) p = 0.f;   // exactly 0 whatever the scale
      psum += p;
      lds_p[my_h * kStep + my_pos[c]] = (uint16_t)(Elem<false>::pack2(p, 0.f) & 0xFFFFu);
    }
    l_run = fmaf(l_run, alpha, psum);
    const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0ull;
    if (rescale && publisher) lds_alpha[my_h] = alpha;
    // the wave's own LDS accesses complete in order; the fence keeps the
    // compiler from moving the reads below ahead of the writes above
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // ---- V: in-lane 8x8 transpose (positions x dims), then next V loads ----
    uint4 vt[8];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      uint32_t vw[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        vw[j] = w == 0 ? vreg[j].x : w == 1 ? vreg[j].y : w == 2 ? vreg[j].z : vreg[j].w;
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
        issue_v_loads<false, D>(vreg, v_cache + next_off, kg, r, next_last, row_bytes);
      else
        issue_v_loads<true, D>(vreg, v_cache + next_off, kg, r, next_last, row_bytes);
    }

    // ---- O = alpha * O + P . V for every head of the group ----
#pragma unroll
    for (int h = 0; h < G; ++h) {
      // probabilities of positions 4*kg .. +4 and 16 + 4*kg .. +4, as pairs
      const uint2 plo = *reinterpret_cast<const uint2*>(lds_p + h * kStep + 4 * kg);
      const uint2 phi = *reinterpret_cast<const uint2*>(lds_p + h * kStep + 16 + 4 * kg);
      if (rescale) {
        const float al = lds_alpha[h];
#pragma unroll
        for (int jd = 0; jd < 8; ++jd) acc[h][jd] *= al;
      }
#pragma unroll
      for (int jd = 0; jd < 8; ++jd) {
        float o = dot2_bf16(vt[jd].x, plo.x, acc[h][jd]);
        o = dot2_bf16(vt[jd].y, plo.y, o);
        o = dot2_bf16(vt[jd].z, phi.x, o);
        acc[h][jd] = dot2_bf16(vt[jd].w, phi.y, o);
      }
    }
    // the next step's writes must not overtake these reads
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }

  // ---- totals: the sum of head my_h over the lanes that share it; O over the
  // four position groups ----
  l_run += dpp_partner<kDppQuadXor1>(l_run);
  if (G <= 4) l_run += dpp_partner<kDppQuadXor2>(l_run);
  if (G <= 2) l_run += dpp_partner<kDppHalfMirror>(l_run);
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
#pragma unroll
  for (int h = 0; h < G; ++h)
#pragma unroll
    for (int jd = 0; jd < 8; ++jd) {
      float o = acc[h][jd];
      o += __shfl_xor(o, 16, 64);
      o += __shfl_xor(o, 32, 64);
      acc[h][jd] = o;
    }

  // ---- hand over in the layout the MFMA path leaves: lane (r = head, kg)
  // holds O[head r][dim 32*kg + 8*e + jd] in acc_out[jd][e] ----
  if (kg == 0) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float4* dst = reinterpret_cast<float4*>(lds_o + h * D + 8 * r);
      dst[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
      dst[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
    }
  }
  if (publisher) {
    lds_ml[2 * my_h] = m_run;
    lds_ml[2 * my_h + 1] = l_run;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int hr = min(r, G - 1);   // padding lanes read a real head and are ignored later
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float4* src = reinterpret_cast<const float4*>(lds_o + hr * D + 32 * kg + 8 * e);
    const float4 x = src[0], y = src[1];
    acc_out[0][e] = x.x; acc_out[1][e] = x.y; acc_out[2][e] = x.z; acc_out[3][e] = x.w;
    acc_out[4][e] = y.x; acc_out[5][e] = y.y; acc_out[6][e] = y.z; acc_out[7][e] = y.w;
  }
  m_out = lds_ml[2 * hr];
  l_out = lds_ml[2 * hr + 1];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// Normalised bf16 result of a whole sequence straight to `out`.
template <int D, bool F16>
__device__ __forceinline__ void write_output(const DecodeArgs& a, int b, int kvh, int lane,
                                             const f32x4 (&acc)[8], float l_run) {
  using H = HeadDim<D>;
  const int r = lane & 15, kg = lane >> 4;
  // at head_dim 64 only k-groups 0 and 1 hold real dims
  if (r >= a.group || 32 * kg >= D) return;
  const int head = kvh * a.group + r;
  const float inv = 1.0f / (l_run + 1e-9f);
  uint4* orow = a.out + ((int64_t)b * a.num_heads + head) * H::kPieces + 4 * kg;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    uint4 o;
    o.x = Elem<F16>::pack2(acc[0][e] * inv, acc[1][e] * inv);
    o.y = Elem<F16>::pack2(acc[2][e] * inv, acc[3][e] * inv);
    o.z = Elem<F16>::pack2(acc[4][e] * inv, acc[5][e] * inv);
    o.w = Elem<F16>::pack2(acc[6][e] * inv, acc[7][e] * inv);
    orow[e] = o;
  }
}

// Unnormalised partial (D f32 per head) + (max, sum) to slot `slot` of the workspace.
template <int D>
__device__ __forceinline__ void write_partial(const DecodeArgs& a, int64_t slot, int kvh, int lane,
                                              const f32x4 (&acc)[8], float m_run, float l_run) {
  const int r = lane & 15, kg = lane >> 4;
  if (r >= a.group || 32 * kg >= D) return;
  const int64_t row = slot * a.num_heads + kvh * a.group + r;
  float4* prow = reinterpret_cast<float4*>(a.part_o + row * D + 32 * kg);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    prow[2 * e] = make_float4(acc[0][e], acc[1][e], acc[2][e], acc[3][e]);
    prow[2 * e + 1] = make_float4(acc[4][e], acc[5][e], acc[6][e], acc[7][e]);
  }
  if (kg == 0) reinterpret_cast<float2*>(a.part_ml)[row] = make_float2(m_run, l_run);
}

// compute_segment, then: `direct` (the segment is the whole sequence) -> out,
// otherwise -> partial slot `slot`.
template <int D, bool F16, int VG = 0>
__device__ __forceinline__ void run_segment(const DecodeArgs& a, uint4* lds, int b, int kvh,
                                            int t0, int t1, int64_t slot, bool direct,
                                            int lane) {
  f32x4 acc[8];
  float m_run, l_run;
  if constexpr (VG > 0) compute_segment_valu<VG>(a, lds, b, kvh, t0, t1, lane, acc, m_run, l_run);
  else compute_segment<D, F16>(a, lds, b, kvh, t0, t1, lane, acc, m_run, l_run);
  if (direct) write_output<D, F16>(a, b, kvh, lane, acc, l_run);
  else write_partial<D>(a, slot, kvh, lane, acc, m_run, l_run);
}

// Fixed-chunk split: grid.x = batch * max_chunks, grid.y = num_kv_heads / NW,
// block = NW * 64.  Workgroup (b, c) owns positions [c*chunk, (c+1)*chunk) of
// sequence b; partial slot = b * max_chunks + c.
template <int NW, int D, bool F16>
__global__ __launch_bounds__(NW * 64) void paged_decode_splitk_kernel(DecodeArgs a, int chunk,
                                                                      int max_chunks) {
  __shared__ uint4 k_tile[NW][kStep * HeadDim<D>::kLdsRowPieces];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int b = blockIdx.x / max_chunks;
  const int c = blockIdx.x - b * max_chunks;
  // A length beyond what the block table can describe is clamped to it.
  const int ctx = min(a.context_lens[b], a.max_blocks * a.block_size);
  const int t0 = c * chunk;
  if (t0 >= ctx) return;  // also every chunk of an empty sequence
  const int t1 = min(ctx, t0 + chunk);
  const bool direct = ctx <= chunk;
  run_segment<D, F16>(a, k_tile[wave], b, blockIdx.y * NW + wave, t0, t1,
                      (int64_t)b * max_chunks + c, direct, lane);
}

// Whole-sequence split: every sequence is finished inside one workgroup, so
// there is no workspace and no second pass.  grid.x = batch * (num_kv_heads /
// hpw), block = NW * 64.  Workgroup (b, head group hg) owns `hpw` KV heads of
// sequence b; its NW waves are hpw heads x NW / hpw parts: wave w takes head
// hg * hpw + w % hpw and the (w / hpw)-th of NW / hpw equal runs of the
// sequence's 32-position steps.  The parts of a head meet through LDS (each
// wave's K tile is free by then and exactly holds its 34 floats per lane) and
// the wave of part 0 merges them and writes the output.  Meant for batches of
// similar lengths: a workgroup's time follows its sequence's length.
// VG > 0 selects the vector-ALU measurement variant for exactly VG query heads
// per KV head (head_dim 128, bf16 only).
template <int NW, int D, bool F16, int VG = 0>
__global__ __launch_bounds__(NW * 64) void paged_decode_whole_kernel(DecodeArgs a, int hpw) {
  using H = HeadDim<D>;
  __shared__ uint4 k_tile[NW][kStep * H::kLdsRowPieces];
  constexpr int kLanesWithDims = D / 32 * 16;   // lanes whose k-group holds real dims
  static_assert(sizeof(uint4) * kStep * H::kLdsRowPieces >= 34 * kLanesWithDims * sizeof(float),
                "a wave's K tile must hold its partial");
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int parts = NW / hpw;
  const int groups = a.num_kv_heads / hpw;
  const int b = blockIdx.x / groups;
  const int hg = blockIdx.x - b * groups;
  const int part = wave / hpw;
  const int kvh = hg * hpw + (wave - part * hpw);
  const int ctx = min(max(as_constant(a.context_lens)[b], 0), a.max_blocks * a.block_size);
  const int steps = (ctx + kStep - 1) / kStep;
  const int s0 = (int)((int64_t)part * steps / parts);
  const int s1 = (int)((int64_t)(part + 1) * steps / parts);

  f32x4 acc[8];
#pragma unroll
  for (int jd = 0; jd < 8; ++jd) acc[jd] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = kNegBig, l_run = 0.f;
  if (s1 > s0) {
    if constexpr (VG > 0)
      compute_segment_valu<VG>(a, k_tile[wave], b, kvh, s0 * kStep, min(ctx, s1 * kStep), lane,
                               acc, m_run, l_run);
    else
      compute_segment<D, F16>(a, k_tile[wave], b, kvh, s0 * kStep, min(ctx, s1 * kStep), lane,
                              acc, m_run, l_run);
  }
  if (parts > 1) {
    // value v of lane l at float v * kLanesWithDims + l of the wave's tile
    const bool holds_dims = lane < kLanesWithDims;
    __syncthreads();   // every wave is done reading its K tile
    if (part > 0 && holds_dims) {
      float* mine = reinterpret_cast<float*>(k_tile[wave]) + lane;
#pragma unroll
      for (int jd = 0; jd < 8; ++jd)
#pragma unroll
        for (int e = 0; e < 4; ++e) mine[(4 * jd + e) * kLanesWithDims] = acc[jd][e];
      mine[32 * kLanesWithDims] = m_run;
      mine[33 * kLanesWithDims] = l_run;
    }
    __syncthreads();
    if (part > 0) return;
    if (holds_dims) {
      for (int p = 1; p < parts; ++p) {
        const float* theirs = reinterpret_cast<const float*>(k_tile[wave + p * hpw]) + lane;
        const float m_p = theirs[32 * kLanesWithDims], l_p = theirs[33 * kLanesWithDims];
        const float m_new = fmaxf(m_run, m_p);
        const float keep = __builtin_amdgcn_exp2f((m_run - m_new) * a.scale_log2e);
        const float w = __builtin_amdgcn_exp2f((m_p - m_new) * a.scale_log2e);
        m_run = m_new;
        l_run = fmaf(l_run, keep, w * l_p);
#pragma unroll
        for (int jd = 0; jd < 8; ++jd)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            acc[jd][e] = fmaf(acc[jd][e], keep, w * theirs[(4 * jd + e) * kLanesWithDims]);
      }
    }
  }
  write_output<D, F16>(a, b, kvh, lane, acc, l_run);
}

// Inclusive prefix sum over the 64 lanes of a wave with DPP moves: a
// Hillis-Steele scan inside each row of 16 lanes (a lane without a source in
// its row adds 0), then the last lane of row 0 / row 2 is added to rows 1 / 3
// (row_bcast:15) and the last lane of row 1 to rows 2 and 3 (row_bcast:31).
__device__ __forceinline__ int wave_inclusive_scan(int x) {
  x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, false);  // row_shr:1
  x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, false);  // row_shr:2
  x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, false);  // row_shr:4
  x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, false);  // row_shr:8
  x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);  // row_bcast:15 -> rows 1, 3
  x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);  // row_bcast:31 -> rows 2, 3
  return x;
}

// Balanced split: the 32-position steps of all sequences, laid end to end in
// batch order, are cut into `num_wgs` equal runs of `S` steps (at least
// `min_steps`); workgroup g owns steps [g*S, (g+1)*S) whatever sequences they
// belong to.  A run that crosses a sequence boundary is processed as one
// segment per sequence.  The segment of (workgroup g, sequence b) uses partial
// slot g + b, which is unique because g and b only grow along the runs; the
// slots of one sequence are consecutive.  Every workgroup derives the cut from
// context_lens itself (a wave-wide prefix sum over the batch), so the host
// never needs the lengths.  Workgroup 0 also leaves the exclusive prefix sums
// (steps before each sequence, total at [batch]) in `prefix` for the combine
// pass.  grid.x = num_wgs, grid.y = num_kv_heads / NW, block = NW * 64.
template <int NW, int D, bool F16, int VG = 0>
__global__ __launch_bounds__(NW * 64) void paged_decode_balanced_kernel(DecodeArgs a, int batch,
                                                                        int num_wgs,
                                                                        int min_steps,
                                                                        int32_t* prefix) {
  __shared__ uint4 k_tile[NW][kStep * HeadDim<D>::kLdsRowPieces];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int g = blockIdx.x;
  const int cap = a.max_blocks * a.block_size;
  const bool writer = g == 0 && blockIdx.y == 0 && wave == 0;

  auto ctx_of = [&](int idx) { return idx < batch ? min(max(a.context_lens[idx], 0), cap) : 0; };
  auto steps_of = [&](int idx) { return (ctx_of(idx) + kStep - 1) / kStep; };

  // One pass over the batch, 64 sequences at a time: total number of steps,
  // and for the first kKeep groups the per-lane (steps, steps before) pairs are
  // kept so that locating the start below needs no second read.
  constexpr int kKeep = 4;
  int kept_ctx[kKeep], kept_excl[kKeep];
#pragma unroll
  for (int k = 0; k < kKeep; ++k) kept_ctx[k] = kept_excl[k] = 0;
  int total = 0, total_kept = 0;
#pragma unroll
  for (int k = 0; k < kKeep; ++k) {
    if (k * 64 < batch) {
      kept_ctx[k] = ctx_of(k * 64 + lane);
      const int n = (kept_ctx[k] + kStep - 1) / kStep;
      const int incl = wave_inclusive_scan(n);
      kept_excl[k] = total + incl - n;
      if (writer && k * 64 + lane < batch) prefix[k * 64 + lane] = kept_excl[k];
      total += __builtin_amdgcn_readlane(incl, 63);
    }
  }
  total_kept = total;
  for (int base = kKeep * 64; base < batch; base += 64) {
    const int n = steps_of(base + lane);
    const int incl = wave_inclusive_scan(n);
    if (writer && base + lane < batch) prefix[base + lane] = total + incl - n;
    total += __builtin_amdgcn_readlane(incl, 63);
  }
  if (writer && lane == 0) prefix[batch] = total;
  const int run = max((total + num_wgs - 1) / num_wgs, min_steps);
  const int start = g * run;
  if (start >= total) return;
  const int end = min(total, start + run);

  // the sequence that holds step `start`, the steps before it and its length
  int b = batch, before = total, first_ctx = -1;
  bool found = false;
#pragma unroll
  for (int k = 0; k < kKeep; ++k) {
    const int n = (kept_ctx[k] + kStep - 1) / kStep;
    const unsigned long long hit =
        __ballot(!found && n > 0 && kept_excl[k] <= start && start < kept_excl[k] + n);
    if (hit != 0ull) {
      const int src = __builtin_ctzll(hit);
      b = k * 64 + src;
      before = __shfl(kept_excl[k], src, 64);
      first_ctx = __shfl(kept_ctx[k], src, 64);
      found = true;
    }
  }
  if (!found) {
    int running = total_kept;
    for (int base = kKeep * 64; base < batch; base += 64) {
      const int n = steps_of(base + lane);
      const int incl = wave_inclusive_scan(n);
      const int excl = running + incl - n;
      const unsigned long long hit = __ballot(n > 0 && excl <= start && start < excl + n);
      if (hit != 0ull) {
        const int src = __builtin_ctzll(hit);
        b = base + src;
        before = __shfl(excl, src, 64);
        break;
      }
      running += __builtin_amdgcn_readlane(incl, 63);
    }
  }
  b = __builtin_amdgcn_readfirstlane(b);
  before = __builtin_amdgcn_readfirstlane(before);
  first_ctx = __builtin_amdgcn_readfirstlane(first_ctx);

  // Walk the run.  The guards (b inside the batch, pos not before the
  // sequence) cannot fire when the prefix sums are right; they keep every
  // index in range regardless.
  // Every quantity of the walk is wave-uniform; readfirstlane says so, so
  // that lengths, page lookups and address arithmetic stay on the scalar unit.
  int pos = start;
  while (pos < end && b < batch && pos >= before) {
    const int sb = __builtin_amdgcn_readfirstlane(b);
    // the first sequence's length is already in registers from the scan
    const int ctx = __builtin_amdgcn_readfirstlane(
        first_ctx >= 0 ? first_ctx : min(max(as_constant(a.context_lens)[sb], 0), cap));
    first_ctx = -1;
    const int nb = (ctx + kStep - 1) / kStep;
    if (pos >= before + nb) {  // empty sequence, or this one is finished
      before += nb;
      b = sb + 1;
      continue;
    }
    const int seg_end = min(end, before + nb);
    const int t0 = __builtin_amdgcn_readfirstlane((pos - before) * kStep);
    const int t1 = __builtin_amdgcn_readfirstlane(min(ctx, (seg_end - before) * kStep));
    const bool direct = pos == before && seg_end == before + nb;
    run_segment<D, F16, VG>(a, k_tile[wave], sb, blockIdx.y * NW + wave, t0, t1,
                            (int64_t)(g + sb), direct, lane);
    pos = seg_end;
  }
}

// Merge the partials of one (sequence, query head).  grid = (B, Hq), block = 128
// lanes, one per output dim.  Fixed-chunk mode (prefix == nullptr): the
// partials of sequence b are slots b*max_chunks .. + ceil(ctx/chunk).  Balanced
// mode: they are slots g_first + b .. g_last + b, where g_first..g_last are the
// workgroups whose runs of `run` steps touch the sequence.  A sequence with one
// partial was written by the split kernel itself; an empty one gives zeros.
__global__ __launch_bounds__(kMaxHeadDim) void paged_decode_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const int32_t* __restrict__ context_lens, const int32_t* __restrict__ prefix,
    uint16_t* __restrict__ out, int num_heads, int chunk, int max_chunks, int max_positions,
    int batch, int num_wgs, int min_steps, float scale_log2e, bool f16) {
  const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
  const int head_dim = blockDim.x;
  int nparts;
  int64_t first;
  if (prefix == nullptr) {
    const int ctx = min(context_lens[b], max_positions);
    nparts = ctx <= 0 ? 0 : (ctx + chunk - 1) / chunk;
    first = (int64_t)b * max_chunks;
  } else {
    const int before = prefix[b], nb = prefix[b + 1] - before, total = prefix[batch];
    const int run = max((total + num_wgs - 1) / num_wgs, min_steps);
    const int g_first = before / run;
    nparts = nb <= 0 ? 0 : (before + nb - 1) / run - g_first + 1;
    first = (int64_t)g_first + b;
  }
  if (nparts == 1) return;  // written by the split kernel itself
  uint16_t* o = out + ((int64_t)b * num_heads + h) * head_dim + d;
  if (nparts == 0) {  // empty sequence: 0 / (0 + 1e-9)
    *o = 0;
    return;
  }
  const int64_t base = first * num_heads + h;
  const float2* ml = reinterpret_cast<const float2*>(part_ml);
  // One pass, 8 partials at a time with all their loads issued together, merged
  // with the running-max rescale.
  float m = kNegBig, num = 0.f, den = 0.f;
  for (int c0 = 0; c0 < nparts; c0 += 8) {
    float2 mlv[8];
    float po[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t row = base + (int64_t)min(c0 + i, nparts - 1) * num_heads;
      mlv[i] = ml[row];
      po[i] = part_o[row * head_dim + d];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (c0 + i < nparts) {
        const float m_new = fmaxf(m, mlv[i].x);
        const float keep = __builtin_amdgcn_exp2f((m - m_new) * scale_log2e);
        const float w = __builtin_amdgcn_exp2f((mlv[i].x - m_new) * scale_log2e);
        num = fmaf(num, keep, w * po[i]);
        den = fmaf(den, keep, w * mlv[i].y);
        m = m_new;
      }
    }
  }
  const float res = num / (den + 1e-9f);
  *o = (uint16_t)((f16 ? Elem<true>::pack2(res, 0.f) : Elem<false>::pack2(res, 0.f)) & 0xFFFFu);
}

int round_up(int x, int m) { return (x + m - 1) / m * m; }

// A wave covers at most 16 query heads (the MFMA columns).  A cache head with
// more than that is walked as `rep` virtual KV heads, the smallest count that
// divides the group into parts of at most 16; its K/V rows are then read once
// per virtual head.
int virtual_heads_per_cache_head(int group) {
  int rep = 1;
  while (group % rep != 0 || group / rep > 16) ++rep;
  return rep;
}

// Whole-sequence mode: KV heads per 8-wave workgroup.  As many as still give
// one workgroup per CU (256), so that the split inside a workgroup is no finer
// than needed; it must divide the number of KV heads.
int whole_sequence_heads_per_workgroup(int64_t batch, int num_kv_heads) {
  int hpw = 8;
  while (hpw > 1 && (num_kv_heads % hpw != 0 || batch * (num_kv_heads / hpw) < 256)) hpw /= 2;
  return hpw;
}

// Balanced mode launches at most one workgroup per CU of an MI355X, and never
// gives a workgroup fewer than 4 steps (128 positions): below that the
// partials cost more than the split gains.
constexpr int kMaxBalancedWorkgroups = 256;
constexpr int kMinBalancedSteps = 4;

// Waves per workgroup = KV heads a workgroup covers: the largest of 8, 4, 2, 1
// that divides the number of KV heads.
int waves_per_workgroup(int num_kv_heads) {
  return num_kv_heads % 8 == 0 ? 8 : num_kv_heads % 4 == 0 ? 4 : num_kv_heads % 2 == 0 ? 2 : 1;
}

// Runs (grid.x) of the balanced split.  grid.y = num_kv_heads / waves per
// workgroup head groups walk the same runs, so the cap of one workgroup per CU
// applies to their product.
int balanced_workgroups(int64_t batch, int64_t max_blocks, int64_t block_size, int num_kv_heads) {
  const int head_groups = num_kv_heads / waves_per_workgroup(num_kv_heads);
  const int64_t cap = kMaxBalancedWorkgroups / head_groups > 0
                          ? kMaxBalancedWorkgroups / head_groups : 1;
  const int64_t max_steps = batch * ((max_blocks * block_size + kStep - 1) / kStep);
  const int64_t wgs = (max_steps + kMinBalancedSteps - 1) / kMinBalancedSteps;
  return (int)(wgs < 1 ? 1 : wgs > cap ? cap : wgs);
}

// Workspace layout.  Fixed chunks: slots = batch * max_chunks.  Balanced:
// slots = workgroups + batch, followed by the int32 prefix array [batch + 1].
struct WorkspacePlan {
  int64_t slots;
  int max_chunks;   // fixed-chunk mode only
  int num_wgs;      // balanced mode only
  size_t bytes;
};

bool plan_workspace(int64_t batch, int64_t num_heads, int64_t head_dim, int64_t max_blocks,
                    int64_t block_size, int num_kv_heads, int chunk, WorkspacePlan* plan) {
  if (chunk == 0) {
    plan->num_wgs = balanced_workgroups(batch, max_blocks, block_size, num_kv_heads);
    plan->max_chunks = 0;
    plan->slots = plan->num_wgs + batch;
    const size_t floats = (size_t)plan->slots * num_heads * (head_dim + 2);
    plan->bytes = floats * sizeof(float) + (size_t)(batch + 1) * sizeof(int32_t);
    return batch * ((max_blocks * block_size + kStep - 1) / kStep) <= INT32_MAX;
  }
  const int64_t mc = (max_blocks * block_size + chunk - 1) / chunk;
  if (batch * mc > INT32_MAX) return false;
  plan->num_wgs = 0;
  plan->max_chunks = (int)mc;
  plan->slots = batch * mc;
  plan->bytes = (size_t)plan->slots * num_heads * (head_dim + 2) * sizeof(float);
  return true;
}

}  // namespace

extern "C" int32_t nvj_paged_decode_default_chunk(int32_t batch, int32_t num_kv_heads,
                                                  int32_t max_blocks, int32_t block_size) {
  if (batch <= 0 || num_kv_heads <= 0 || max_blocks <= 0 || block_size <= 0) return 256;
  // One 8-wave workgroup is resident per CU and a launch is fastest at exactly
  // one workgroup per CU (256 on MI355X): the chunk that gives that when every
  // sequence is at full length, if it is at most 2048 positions; else 1024,
  // which keeps ragged batches balanced; never below 128.
  const int64_t positions = (int64_t)batch * max_blocks * block_size;
  int64_t chunk = (positions + 255) / 256;
  if (chunk < 128) chunk = 128;
  if (chunk > 2048) chunk = 1024;
  return round_up((int)chunk, kStep);
}

extern "C" int32_t nvj_paged_decode_whole_sequence_workgroups(int32_t batch, int32_t num_heads,
                                                               int32_t num_kv_heads) {
  if (batch <= 0 || num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0) return 0;
  const int64_t heads =
      (int64_t)num_kv_heads * virtual_heads_per_cache_head(num_heads / num_kv_heads);
  if (batch * heads > INT32_MAX) return 0;
  return batch * ((int)heads / whole_sequence_heads_per_workgroup(batch, (int)heads));
}

extern "C" size_t nvj_paged_decode_workspace_bytes(int32_t batch, int32_t num_heads,
                                                   int32_t head_dim, int32_t max_blocks,
                                                   int32_t block_size, int32_t num_kv_heads,
                                                   int32_t chunk) {
  if (chunk == NVJ_CHUNK_WHOLE_SEQUENCE) return 0;   // finished inside the workgroups
  if (batch <= 0 || num_heads <= 0 || (head_dim != 128 && head_dim != 64) || max_blocks <= 0 ||
      block_size <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || chunk < 0 ||
      chunk % kStep != 0)
    return 0;
  num_kv_heads *= virtual_heads_per_cache_head(num_heads / num_kv_heads);
  WorkspacePlan plan;
  if (!plan_workspace(batch, num_heads, head_dim, max_blocks, block_size, num_kv_heads, chunk,
                      &plan))
    return 0;
  return plan.bytes;
}

extern "C" int nvj_paged_decode_launch_phases(void* stream, const void* q, const void* k_cache,
                                              const void* v_cache, const int32_t* block_tables,
                                              const int32_t* context_lens, void* out,
                                              void* workspace, size_t workspace_bytes,
                                              int32_t batch, int32_t num_heads,
                                              int32_t num_kv_heads, int32_t head_dim,
                                              int32_t block_size, int32_t max_blocks,
                                              int32_t num_blocks, float scale, int32_t chunk,
                                              int32_t dtype, uint32_t phases) {
  if (dtype != NVJ_DTYPE_BF16 && dtype != NVJ_DTYPE_F16) return NVJ_ERR_BAD_DTYPE;
  const bool f16 = dtype == NVJ_DTYPE_F16;
  const bool whole = chunk == NVJ_CHUNK_WHOLE_SEQUENCE;
  if (batch < 0 || num_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || block_size <= 0 ||
      max_blocks < 0 || num_blocks <= 0 || (chunk < 0 && !whole))
    return NVJ_ERR_BAD_SHAPE;
  if (num_heads % num_kv_heads != 0) return NVJ_ERR_BAD_SHAPE;
  if ((head_dim != 128 && head_dim != 64) || block_size % kStep != 0 ||
      (!whole && chunk % kStep != 0))
    return NVJ_ERR_UNSUPPORTED;
  const int cache_kv_heads = num_kv_heads;
  const int kv_rep = virtual_heads_per_cache_head(num_heads / num_kv_heads);
  if ((int64_t)num_kv_heads * kv_rep > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  num_kv_heads *= kv_rep;   // from here on: the heads as the kernels walk them
  const int group = num_heads / num_kv_heads;
  if ((int64_t)max_blocks * block_size > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  if (!(scale >= 0.f)) return NVJ_ERR_BAD_SHAPE;   // the running max assumes a non-negative scale
  if (batch == 0) return NVJ_OK;
  if (!q || !k_cache || !v_cache || !context_lens || !out) return NVJ_ERR_NULL_POINTER;
  if (max_blocks > 0 && !block_tables) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_cache) |
       reinterpret_cast<uintptr_t>(v_cache) | reinterpret_cast<uintptr_t>(out) |
       (whole ? 0 : reinterpret_cast<uintptr_t>(workspace))) & 15u)   // unused in whole mode
    return NVJ_ERR_WORKSPACE;
  // the vector-ALU measurement variant exists for one shape family only
  const bool valu = (phases & NVJ_PHASE_VALU_PRODUCTS) != 0;
  if (valu && (head_dim != 128 || f16 || kv_rep != 1 || (group != 4 && group != 8) ||
               num_kv_heads % 8 != 0 || chunk > 0))
    return NVJ_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);

  DecodeArgs a;
  a.q = static_cast<const uint4*>(q);
  a.k_cache = static_cast<const char*>(k_cache);
  a.v_cache = static_cast<const char*>(v_cache);
  a.block_tables = block_tables;
  a.context_lens = context_lens;
  a.out = static_cast<uint4*>(out);
  a.part_o = nullptr;
  a.part_ml = nullptr;
  a.num_heads = num_heads;
  a.num_kv_heads = num_kv_heads;
  a.group = group;
  a.kv_rep = kv_rep;
  a.cache_kv_heads = cache_kv_heads;
  a.block_size = block_size;
  a.max_blocks = max_blocks;
  a.num_blocks = num_blocks;
  a.scale_log2e = scale * kLog2e;

  if (whole && max_blocks > 0) {
    if ((int64_t)batch * num_kv_heads > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
    if (!(phases & NVJ_PHASE_SPLITK)) return NVJ_OK;   // there is no second pass
    const int hpw = whole_sequence_heads_per_workgroup(batch, num_kv_heads);
    const dim3 grid((unsigned)(batch * (num_kv_heads / hpw)));
    if (valu && group == 4) paged_decode_whole_kernel<8, 128, false, 4><<<grid, dim3(512), 0, s>>>(a, hpw);
    else if (valu) paged_decode_whole_kernel<8, 128, false, 8><<<grid, dim3(512), 0, s>>>(a, hpw);
    else if (head_dim == 128 && !f16) paged_decode_whole_kernel<8, 128, false><<<grid, dim3(512), 0, s>>>(a, hpw);
    else if (head_dim == 128) paged_decode_whole_kernel<8, 128, true><<<grid, dim3(512), 0, s>>>(a, hpw);
    else if (!f16) paged_decode_whole_kernel<8, 64, false><<<grid, dim3(512), 0, s>>>(a, hpw);
    else paged_decode_whole_kernel<8, 64, true><<<grid, dim3(512), 0, s>>>(a, hpw);
    return hipGetLastError() == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
  }

  WorkspacePlan plan = {0, 1, 0, 0};
  int32_t* prefix = nullptr;
  if (max_blocks > 0) {
    if (!plan_workspace(batch, num_heads, head_dim, max_blocks, block_size, num_kv_heads, chunk,
                        &plan))
      return NVJ_ERR_BAD_SHAPE;
    if (!workspace || workspace_bytes < plan.bytes) return NVJ_ERR_WORKSPACE;
    a.part_o = static_cast<float*>(workspace);
    a.part_ml = a.part_o + plan.slots * num_heads * head_dim;
    if (chunk == 0) prefix = reinterpret_cast<int32_t*>(a.part_ml + plan.slots * num_heads * 2);

    if (phases & NVJ_PHASE_SPLITK) {
      const int nw = waves_per_workgroup(num_kv_heads);
      const unsigned gy = (unsigned)(num_kv_heads / nw);
      // one instantiation per (waves per workgroup, head_dim)
#define NVJ_FOR_DTYPE(LAUNCH, NWV, DV) \
  do {                                \
    if (f16) LAUNCH(NWV, DV, true);   \
    else LAUNCH(NWV, DV, false);      \
  } while (0)
#define NVJ_FOR_SHAPE(LAUNCH)                             \
  switch (nw * 1000 + head_dim) {                         \
    case 8128: NVJ_FOR_DTYPE(LAUNCH, 8, 128); break;      \
    case 4128: NVJ_FOR_DTYPE(LAUNCH, 4, 128); break;      \
    case 2128: NVJ_FOR_DTYPE(LAUNCH, 2, 128); break;      \
    case 1128: NVJ_FOR_DTYPE(LAUNCH, 1, 128); break;      \
    case 8064: NVJ_FOR_DTYPE(LAUNCH, 8, 64); break;       \
    case 4064: NVJ_FOR_DTYPE(LAUNCH, 4, 64); break;       \
    case 2064: NVJ_FOR_DTYPE(LAUNCH, 2, 64); break;       \
    default: NVJ_FOR_DTYPE(LAUNCH, 1, 64); break;         \
  }
      if (chunk == 0) {
        const dim3 grid((unsigned)plan.num_wgs, gy);
#define NVJ_LAUNCH_BALANCED(NWV, DV, F16V)                                      \
  paged_decode_balanced_kernel<NWV, DV, F16V><<<grid, dim3(NWV * 64), 0, s>>>( \
      a, batch, plan.num_wgs, kMinBalancedSteps, prefix)
        if (valu && group == 4)
          paged_decode_balanced_kernel<8, 128, false, 4><<<grid, dim3(512), 0, s>>>(
              a, batch, plan.num_wgs, kMinBalancedSteps, prefix);
        else if (valu)
          paged_decode_balanced_kernel<8, 128, false, 8><<<grid, dim3(512), 0, s>>>(
              a, batch, plan.num_wgs, kMinBalancedSteps, prefix);
        else
          NVJ_FOR_SHAPE(NVJ_LAUNCH_BALANCED)
#undef NVJ_LAUNCH_BALANCED
      } else {
        const dim3 grid((unsigned)(batch * plan.max_chunks), gy);
#define NVJ_LAUNCH_FIXED(NWV, DV, F16V)                                                    \
  paged_decode_splitk_kernel<NWV, DV, F16V><<<grid, dim3(NWV * 64), 0, s>>>(a, chunk, \
                                                                             plan.max_chunks)
        NVJ_FOR_SHAPE(NVJ_LAUNCH_FIXED)
#undef NVJ_LAUNCH_FIXED
      }
#undef NVJ_FOR_SHAPE
#undef NVJ_FOR_DTYPE
      if (hipGetLastError() != hipSuccess) return NVJ_ERR_LAUNCH;
    }
  } else {
    chunk = kStep;  // no pages at all: every sequence is empty, combine writes zeros
  }
  if (!(phases & NVJ_PHASE_COMBINE)) return NVJ_OK;
  paged_decode_combine_kernel<<<dim3((unsigned)batch, (unsigned)num_heads), dim3(head_dim), 0, s>>>(
      a.part_o, a.part_ml, context_lens, prefix, static_cast<uint16_t*>(out), num_heads, chunk,
      plan.max_chunks, max_blocks * block_size, batch, plan.num_wgs, kMinBalancedSteps,
      a.scale_log2e, f16);
  return hipGetLastError() == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

extern "C" int nvj_paged_decode_launch(void* stream, const void* q, const void* k_cache,
                                       const void* v_cache, const int32_t* block_tables,
                                       const int32_t* context_lens, void* out, void* workspace,
                                       size_t workspace_bytes, int32_t batch, int32_t num_heads,
                                       int32_t num_kv_heads, int32_t head_dim,
                                       int32_t block_size, int32_t max_blocks,
                                       int32_t num_blocks, float scale, int32_t chunk,
                                       int32_t dtype) {
  return nvj_paged_decode_launch_phases(stream, q, k_cache, v_cache, block_tables, context_lens,
                                        out, workspace, workspace_bytes, batch, num_heads,
                                        num_kv_heads, head_dim, block_size, max_blocks,
                                        num_blocks, scale, chunk, dtype,
                                        NVJ_PHASE_SPLITK | NVJ_PHASE_COMBINE);
}

// ---------------------------------------------------------------------------
// Entry point that allocates nothing: the balanced split with its workspace in
// a file-scope device array instead of caller memory.  The array's name is a
// host-side stand-in; its device address is looked up once per device
// (hipGetSymbolAddress) and only that address is ever handed to a kernel.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[NVJ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];   // per device: address of its copy of `scratch`

// Device address of the current device's copy of `scratch`.
int static_scratch_of_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return NVJ_ERR_LAUNCH;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    // every thread that races here gets the same address from the runtime
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr)
      return NVJ_ERR_LAUNCH;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return NVJ_OK;
}
}  // namespace

extern "C" int nvj_paged_decode_static_launch(void* stream, const void* q, const void* k_cache,
                                              const void* v_cache, const int32_t* block_tables,
                                              const int32_t* context_lens, void* out,
                                              int32_t batch, int32_t num_heads,
                                              int32_t num_kv_heads, int32_t head_dim,
                                              int32_t block_size, int32_t max_blocks,
                                              int32_t num_blocks, float scale, int32_t dtype) {
  void* ws = nullptr;
  if (batch > 0 && max_blocks > 0) {
    const size_t need = nvj_paged_decode_workspace_bytes(batch, num_heads, head_dim, max_blocks,
                                                         block_size, num_kv_heads, 0);
    // need == 0: invalid arguments, which the launch below reports by name
    if (need > NVJ_STATIC_SCRATCH_BYTES) return NVJ_ERR_SCRATCH_LIMIT;
    if (need > 0) {
      const int rc = static_scratch_of_current_device(&ws);
      if (rc != NVJ_OK) return rc;
    }
  }
  return nvj_paged_decode_launch(stream, q, k_cache, v_cache, block_tables, context_lens, out, ws,
                                 ws ? (size_t)NVJ_STATIC_SCRATCH_BYTES : 0, batch, num_heads,
                                 num_kv_heads, head_dim, block_size, max_blocks, num_blocks, scale,
                                 0, dtype);
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
    case NVJ_ERR_SCRATCH_LIMIT:
      return "problem needs more than the library's static scratch (NVJ_STATIC_SCRATCH_BYTES)";
    default: return "unknown error code";
  }
}

extern "C" int nvj_abi_version(void) { return NVJ_ABI_VERSION; }

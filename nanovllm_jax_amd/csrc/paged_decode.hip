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
//   * O^T[dim, qhead] += V^T . P^T with 16 MFMAs: P enters twice, as its values
//     rounded to the cache's 16-bit type and as the rest of that rounding.
// Loads for step i+1 are issued before the arithmetic of step i.
//
// In the first two modes the partial (unnormalised O, running max, running
// sum) of every segment goes to the workspace and the combine kernel merges the
// segments of a sequence; a sequence that is one segment is written directly.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "launch.h"
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
  // the two values a packed pair stands for
  static __device__ __forceinline__ float low_of(uint32_t pair) {
    return __builtin_bit_cast(float, pair << 16);
  }
  static __device__ __forceinline__ float high_of(uint32_t pair) {
    return __builtin_bit_cast(float, pair & 0xFFFF0000u);
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
  static __device__ __forceinline__ float low_of(uint32_t pair) {
    typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
    return (float)__builtin_bit_cast(f16x2, pair)[0];
  }
  static __device__ __forceinline__ float high_of(uint32_t pair) {
    typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
    return (float)__builtin_bit_cast(f16x2, pair)[1];
  }
};

// A pair of fp32 values as two packed pairs of the cache's 16-bit type: the
// rounded values and what the rounding left over, rounded again.  Their sum
// carries 16 (bf16) or 22 (float16) mantissa bits of the fp32 values.
template <bool F16>
__device__ __forceinline__ void pack2_with_rest(float a, float b, uint32_t& main, uint32_t& rest) {
  main = Elem<F16>::pack2(a, b);
  rest = Elem<F16>::pack2(a - Elem<F16>::low_of(main), b - Elem<F16>::high_of(main));
}


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
    // Other lanes read these rows below.  The wave's own LDS accesses complete
    // in order; the fences keep the compiler from moving the reads ahead of the
    // writes (and, at the end of the step, the next writes ahead of the reads).
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
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
    // The probabilities go to the matrix core as two operands of the cache's
    // 16-bit type, the rounded values and the rest of the rounding, so that
    // P.V sees them to 16 bits or more, as good as the fp32 probabilities of the
    // reference's vectorised path (layers/pallas_attention.py:227-236); the
    // second product is free under the K/V stream.
    uint4 pbits, prest;
    pack2_with_rest<F16>(p0[0], p0[1], pbits.x, prest.x);
    pack2_with_rest<F16>(p0[2], p0[3], pbits.y, prest.y);
    pack2_with_rest<F16>(p1[0], p1[1], pbits.z, prest.z);
    pack2_with_rest<F16>(p1[2], p1[3], pbits.w, prest.w);

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
      acc[jd] = Elem<F16>::mfma(vt[jd], prest, acc[jd]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
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

// ---------------------------------------------------------------------------
// Measurement variant: the load stream of a segment and nothing else.  Same
// page walk, same K and V loads (addresses, order, one step fetched ahead) as
// compute_segment, but what arrives is only folded into one word per lane: no
// LDS, no matrix or softmax work.  Timing it against the real kernel shows how
// much of the kernel's time the arithmetic adds on top of the memory stream.
// The "result" is meaningless (and finite).  head_dim 128 only.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void compute_segment_loads_only(const DecodeArgs& a, int b, int kvh,
                                                           int t0, int t1, int lane,
                                                           f32x4 (&acc)[8], float& m_run,
                                                           float& l_run) {
  constexpr int D = 128;
  using H = HeadDim<D>;
  const int r = lane & 15, kg = lane >> 4;
  const int block_size = a.block_size, num_blocks = a.num_blocks;
  const int nsteps = (t1 - t0 + kStep - 1) / kStep;
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
    issue_k_loads<true, D>(kreg, a.k_cache + off, lane, last, row_bytes);
    issue_v_loads<true, D>(vreg, a.v_cache + off, kg, r, last, row_bytes);
  }
#pragma unroll
  for (int jd = 0; jd < 8; ++jd) acc[jd] = f32x4{0.f, 0.f, 0.f, 0.f};
  m_run = 0.f;
  l_run = 0.f;
  uint32_t folded = 0;
  int64_t off_ahead = nsteps > 1 ? step_base(1) : 0;
  for (int step = 0; step < nsteps; ++step) {
    const bool more = step + 1 < nsteps;
    const int64_t next_off = off_ahead;
    int next_last = kStep - 1;
    if (more) next_last = min(kStep, t1 - (t0 + (step + 1) * kStep)) - 1;
    if (step + 2 < nsteps) off_ahead = step_base(step + 2);
#pragma unroll
    for (int i = 0; i < H::kKLoads; ++i) folded ^= kreg[i].x ^ kreg[i].y ^ kreg[i].z ^ kreg[i].w;
#pragma unroll
    for (int j = 0; j < 8; ++j) folded ^= vreg[j].x ^ vreg[j].y ^ vreg[j].z ^ vreg[j].w;
    if (more) {
      if (next_last == kStep - 1) {
        issue_k_loads<false, D>(kreg, a.k_cache + next_off, lane, next_last, row_bytes);
        issue_v_loads<false, D>(vreg, a.v_cache + next_off, kg, r, next_last, row_bytes);
      } else {
        issue_k_loads<true, D>(kreg, a.k_cache + next_off, lane, next_last, row_bytes);
        issue_v_loads<true, D>(vreg, a.v_cache + next_off, kg, r, next_last, row_bytes);
      }
    }
    l_run += 1.0f;
  }
  acc[0][0] = (float)(folded & 0xFFu);
}

// Folds the partial another wave of the workgroup left in its LDS tile into this
// wave's (acc, m_run, l_run): value v of a lane at float v * STRIDE of `theirs`
// (already offset by the lane), v = 4 * jd + e for acc[jd][e], 32 the running
// max, 33 the running sum.  All 34 values are fetched before the first is used:
// read one by one, as the compiler orders them when left alone, the 17 LDS
// round trips of every part follow each other (1.3 us for 3 parts).
template <int STRIDE>
__device__ __forceinline__ void add_partial_from_lds(const float* theirs, float scale_log2e,
                                                     f32x4 (&acc)[8], float& m_run, float& l_run) {
  float t[34];
#pragma unroll
  for (int v = 0; v < 34; ++v) t[v] = theirs[v * STRIDE];
  __builtin_amdgcn_sched_barrier(0);
  const float m_new = fmaxf(m_run, t[32]);
  const float keep = __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2e);
  const float w = __builtin_amdgcn_exp2f((t[32] - m_new) * scale_log2e);
  m_run = m_new;
  l_run = fmaf(l_run, keep, w * t[33]);
#pragma unroll
  for (int jd = 0; jd < 8; ++jd)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[jd][e] = fmaf(acc[jd][e], keep, w * t[4 * jd + e]);
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

// Unnormalised partial (D f32 per head) + (max, sum) to the workspace.  A
// partial record is D + 2 floats of one query head; `rec_base` is the record of
// the first query head of this wave's KV head.
template <int D>
__device__ __forceinline__ void write_partial(const DecodeArgs& a, int64_t rec_base, int lane,
                                              const f32x4 (&acc)[8], float m_run, float l_run) {
  const int r = lane & 15, kg = lane >> 4;
  if (r >= a.group || 32 * kg >= D) return;
  const int64_t row = rec_base + r;
  float4* prow = reinterpret_cast<float4*>(a.part_o + row * D + 32 * kg);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    prow[2 * e] = make_float4(acc[0][e], acc[1][e], acc[2][e], acc[3][e]);
    prow[2 * e + 1] = make_float4(acc[4][e], acc[5][e], acc[6][e], acc[7][e]);
  }
  if (kg == 0) reinterpret_cast<float2*>(a.part_ml)[row] = make_float2(m_run, l_run);
}

// Fixed-chunk split: grid.x = batch * max_chunks, grid.y = num_kv_heads / NW,
// block = NW * 64.  Workgroup (b, c) owns positions [c*chunk, (c+1)*chunk) of
// sequence b; partial slot = b * max_chunks + c holds all query heads.
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
  const int kvh = blockIdx.y * NW + wave;
  f32x4 acc[8];
  float m_run, l_run;
  compute_segment<D, F16>(a, k_tile[wave], b, kvh, t0, t1, lane, acc, m_run, l_run);
  if (ctx <= chunk) write_output<D, F16>(a, b, kvh, lane, acc, l_run);
  else write_partial<D>(a, ((int64_t)b * max_chunks + c) * a.num_heads + kvh * a.group, lane, acc,
                        m_run, l_run);
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
// VG < 0 selects the loads-only measurement variant; VG > 0 selects the
// vector-ALU measurement variant for exactly VG query heads
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
    else if constexpr (VG < 0)
      compute_segment_loads_only(a, b, kvh, s0 * kStep, min(ctx, s1 * kStep), lane, acc, m_run,
                                 l_run);
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
        add_partial_from_lds<kLanesWithDims>(
            reinterpret_cast<const float*>(k_tile[wave + p * hpw]) + lane, a.scale_log2e, acc, m_run,
            l_run);
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

// Maximum over the 64 lanes of a wave, wave-uniform, with the same DPP moves (a
// lane without a source keeps its own value).
__device__ __forceinline__ int wave_max(int x) {
  x = max(x, __builtin_amdgcn_update_dpp(x, x, 0x111, 0xF, 0xF, false));
  x = max(x, __builtin_amdgcn_update_dpp(x, x, 0x112, 0xF, 0xF, false));
  x = max(x, __builtin_amdgcn_update_dpp(x, x, 0x114, 0xF, 0xF, false));
  x = max(x, __builtin_amdgcn_update_dpp(x, x, 0x118, 0xF, 0xF, false));
  x = max(x, __builtin_amdgcn_update_dpp(x, x, 0x142, 0xA, 0xF, false));
  x = max(x, __builtin_amdgcn_update_dpp(x, x, 0x143, 0xC, 0xF, false));
  return __builtin_amdgcn_readlane(x, 63);
}

// ---------------------------------------------------------------------------
// Balanced split: one launch for any mix of lengths.
//
// A workgroup is 8 waves = `hpw` KV heads x R = 8 / hpw parts (hpw is 4, 2 or
// 1 by the size of the launch, see balanced_heads_per_workgroup on the host side).
// The unit of work is a "row step": one 32-position step of one row, a row
// being (sequence b, head group hg of hpw KV heads).  All row steps, ordered
// by (b, hg, step), form one axis of length T = (num_kv_heads / hpw) * sum of
// steps.  The axis is cut into `nsub` sub-runs of equal length to within one
// step (`Cut` below): nsub = workgroups x R when there is at least one step for
// each, fewer otherwise.  Sub-run j belongs to workgroup j / R, part j % R, and
// is walked by the hpw waves of that part, one KV head each.  Every wave
// derives the cut from context_lens itself (a wave-wide prefix sum over the
// batch), so the host never needs the lengths.
//
// A sub-run that covers a whole row writes the output directly.  Otherwise a
// row is shared by several sub-runs; the piece of row `row` in sub-run j is a
// segment and owns partial slot j + row (unique, because j and row only grow
// along the axis, and consecutive within a row).  When the whole run of a
// workgroup lies inside one row, its parts are first merged through LDS (a
// wave's K tile is free by then) and part 0 writes one partial for all of
// them; the slots of the other parts stay unused, which the merging wave knows
// from the cut.
//
// Merge without a second launch: `counters` holds one int32 per (sequence, KV
// head), zero between launches.  A wave that has written partials for a row
// adds the number of sub-runs they stand for; the wave whose addition
// completes the row's count (the number of sub-runs that touch the row, known
// from the cut) merges the row's partials (in an order fixed by the cut alone,
// so that the result does not depend on who merges), writes the output and puts
// the counter back to zero.  Nothing ever waits for another workgroup.
// ---------------------------------------------------------------------------

// Sequences whose (length, steps before) pairs every wave keeps in registers
// after its one pass over the lengths; further ones are read again when needed.
constexpr int kKeptSequences = 256;

// Whole rows in the order of the batch, several rows per workgroup: only when
// no workgroup gets more than 1 + 8/256 of the mean (beyond that the order by
// length, which the caller's tolerance applies to, usually does better).
constexpr int kWholeRowTightTolerance = 8;
// The whole-row layout is offered for launches of up to this many workgroups
// (every wave checks the deal of all of them, 64 per pass).
constexpr int kMaxWholeRowWorkgroups = 256;

// The cut of the axis: sub-run j covers the axis positions whose unit
// (position >> shift) lies in [floor(j * units / nsub), floor((j+1) * units / nsub)).
// shift is 0 unless the axis is so long that units * nsub would not fit 31 bits
// (the host picks it from the largest axis the shapes allow).  Every sub-run
// holds at least one position.
struct Cut {
  int axis;    // row steps in all
  int units;   // ceil(axis >> shift)
  int nsub;    // sub-runs in use, 1 <= nsub <= units
  int shift;
  __device__ __forceinline__ int start_of(int j) const {
    const uint32_t u = (uint32_t)j * (uint32_t)units / (uint32_t)nsub;
    return min(axis, (int)(u << shift));
  }
  __device__ __forceinline__ int subrun_of(int x) const {
    return (int)((((uint32_t)(x >> shift) + 1u) * (uint32_t)nsub - 1u) / (uint32_t)units);
  }
};

// Record (see write_partial) of query head 0 of KV head `h_in_row` of a slot.
__device__ __forceinline__ int64_t balanced_record(const DecodeArgs& a, int64_t slot, int hpw,
                                                   int h_in_row) {
  return (slot * hpw + h_in_row) * a.group;
}

// Partials of the balanced split travel between workgroups of one launch, and
// workgroups on different XCDs do not share an L2.  They are therefore written
// and read with device-scope accesses (cache policy sc1: written through to,
// and read from, the point where the XCDs meet), ordered against the row's
// counter by waiting for the stores to be acknowledged.  No cache-wide
// write-back or invalidate is ever issued; those stall the K/V stream of every
// other wave on the XCD.  The accesses are 16-byte buffer instructions over a
// window that starts at a wave-uniform address.
//
// Layout of the partial of one (slot, KV head), chosen so that every store
// instruction of a wave writes one contiguous run: 16-byte piece i (0..7) of
// lane (r = query head, kg = dim group) sits at piece index
// i * (D/32 * G) + kg * G + r.  Piece 2e holds acc[0..3][e], piece 2e+1
// acc[4..7][e] of that lane.  The (max, sum) pairs follow the record order.
typedef __attribute__((ext_vector_type(4))) float vfloat4;
typedef __attribute__((ext_vector_type(2))) float vfloat2;
typedef __attribute__((ext_vector_type(4))) unsigned int vuint4;
typedef __attribute__((ext_vector_type(2))) unsigned int vuint2;
constexpr int kDeviceScope = 16;   // buffer cache policy: sc1

__device__ __forceinline__ __amdgpu_buffer_rsrc_t device_window(const void* base, int64_t bytes) {
  const int n = (int)(bytes < 0x7fffffff ? bytes : 0x7fffffff);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, n, 0x00020000);
}

template <int D>
__device__ __forceinline__ void write_partial_coherent(const DecodeArgs& a, int64_t rec_base,
                                                       int lane, const f32x4 (&acc)[8],
                                                       float m_run, float l_run) {
  constexpr int KG = D / 32;
  const int r = lane & 15, kg = lane >> 4;
  if (r >= a.group || kg >= KG) return;
  const __amdgpu_buffer_rsrc_t wo =
      device_window(a.part_o + rec_base * D, (int64_t)a.group * D * sizeof(float));
  const int lane_off = (kg * a.group + r) * 16, piece_stride = KG * a.group * 16;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const vfloat4 lo = {acc[0][e], acc[1][e], acc[2][e], acc[3][e]};
    const vfloat4 hi = {acc[4][e], acc[5][e], acc[6][e], acc[7][e]};
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(vuint4, lo), wo,
                                           lane_off + 2 * e * piece_stride, 0, kDeviceScope);
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(vuint4, hi), wo,
                                           lane_off + (2 * e + 1) * piece_stride, 0, kDeviceScope);
  }
  if (kg == 0) {
    const __amdgpu_buffer_rsrc_t wm =
        device_window(a.part_ml + rec_base * 2, (int64_t)a.group * 2 * sizeof(float));
    const vfloat2 ml = {m_run, l_run};
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(vuint2, ml), wm, r * 8, 0,
                                          kDeviceScope);
  }
}

// All earlier stores of this wave have been acknowledged (and no later memory
// operation is moved ahead of this point by the compiler).
__device__ __forceinline__ void wait_for_stores() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// arrive: the wave has written its partials of row [r0, r1) (row steps on the
// axis) of (sequence b, KV head kvh), standing for `n` sub-runs, and publishes
// them.  merge_row: all partials of the row are there; merge them and write the
// output.  `lds` is the wave's own tile (free at that point).
//
// The merge keeps the chain of dependent memory round trips short: which slots
// hold a partial is computed from the cut, not read; the (max, sum) pairs of up
// to 64 slots are fetched by loads issued together and spread to the lanes
// through LDS; the accumulators of four partials are in flight at once.
// Returns true when this arrival completed the row: the caller then owes the
// row its merge (merge_row), at a time of its choosing.
__device__ __forceinline__ bool arrive(const DecodeArgs& a, int32_t* counters, int b, int kvh,
                                       int r0, int r1, const Cut& cut, int n, int lane) {
  // the partial stores of every lane have reached the device before the count does
  wait_for_stores();
  // word 0 of the counter region is the stale flag, the counters follow
  int32_t* counter = counters + 1 + (int64_t)b * a.num_kv_heads + kvh;
  int old = 0;
  if (lane == 0)
    old = __hip_atomic_fetch_add(counter, n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  old = __builtin_amdgcn_readfirstlane(old);
  const int expected = cut.subrun_of(r1 - 1) - cut.subrun_of(r0) + 1;
  if (old < 0 || old + n > expected) {
    // The counter did not start at zero: the region was never cleared, an earlier
    // launch on it was cut short, or two launches overlap on it.  This row's
    // output is lost; say so where the host can see it and put the counter
    // back, so that a launch after this one starts from zero again.
    if (lane == 0) {
      __hip_atomic_store(counters, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return false;
  }
  if (old + n != expected) return false;
  // last to arrive: every other partial of the row was acknowledged before its
  // writer's count, which this wave has just seen
  asm volatile("" ::: "memory");
  if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}

// x of the lane n places further on in its row of 16 lanes (wrapping around)
template <int N>
__device__ __forceinline__ float row_rotate(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 | N, 0xf, 0xf, false));
}

template <int D, bool F16>
__device__ __forceinline__ void merge_row(const DecodeArgs& a, uint4* lds, int b, int kvh,
                                          int hpw, int r0, int r1, const Cut& cut, int lane) {
  using H = HeadDim<D>;
  // slots whose (max, sum) pairs fit the wave's tile at 16 heads x 8 bytes each
  constexpr int kSlots = (kStep * H::kLdsRowPieces * 16) / 128 >= 64 ? 64 : 32;
  static_assert(kStep * H::kLdsRowPieces * 16 >= kSlots * 128 + kSlots, "room for the slot list");
  constexpr int KG = D / 32;
  const int parts = 8 / hpw;
  const int first = cut.subrun_of(r0);
  const int expected = cut.subrun_of(r1 - 1) - first + 1;
  const int hg = kvh / hpw;
  const int rows_per_seq = a.num_kv_heads / hpw;
  const int64_t slot0 = (int64_t)first + (int64_t)b * rows_per_seq + hg;
  // A row of 16 lanes has room for 16 query heads; with fewer, the row is cut
  // into 16 / gp lane groups of gp >= group lanes (gp a power of two) and every
  // lane group merges partials of its own, so that 4 * 16 / gp partials are in
  // flight at once; the lane groups are added up at the end.  Lanes of padding
  // heads / padding dims read a real record and drop it later.
  const int gp = a.group > 8 ? 16 : a.group > 4 ? 8 : a.group > 2 ? 4 : a.group > 1 ? 2 : 1;
  const int lane_groups = 16 / gp;
  const int lg = (lane & 15) / gp;                        // this lane's group
  const int r = min((lane & 15) - lg * gp, a.group - 1);  // its query head
  const int kg = (32 * (lane >> 4) < D) ? (lane >> 4) : 0;
  const int64_t rec0 = balanced_record(a, slot0, hpw, kvh - hg * hpw);   // slot0, head 0
  const int64_t rec_stride = (int64_t)hpw * a.group;                     // per slot
  const __amdgpu_buffer_rsrc_t wm = device_window(
      a.part_ml + rec0 * 2, ((int64_t)(expected - 1) * rec_stride + a.group) * 2 * sizeof(float));
  const __amdgpu_buffer_rsrc_t wo = device_window(
      a.part_o + rec0 * D, ((int64_t)(expected - 1) * rec_stride + a.group) * D * sizeof(float));
  const int slot_bytes = (int)rec_stride * D * (int)sizeof(float);
  const int lane_off = (kg * a.group + r) * 16, piece_stride = KG * a.group * 16;
  vfloat2* lds_ml = reinterpret_cast<vfloat2*>(lds);   // [kSlots][16 heads]
  uint8_t* lds_list = reinterpret_cast<uint8_t*>(lds_ml + kSlots * 16);   // [kSlots]
  f32x4 acc[8];
#pragma unroll
  for (int jd = 0; jd < 8; ++jd) acc[jd] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = kNegBig, l_run = 0.f;
  for (int base = 0; base < expected; base += kSlots) {
    // Which of the slots base .. base + kSlots - 1 hold a partial follows from the
    // cut: lane L answers for slot base + L.  A workgroup whose whole run lies
    // inside this row merged its parts in LDS and wrote one partial, in the slot
    // of its part 0; any other workgroup wrote one per sub-run.
    const int count = min(kSlots, expected - base);
    const int j = first + base + lane;
    const int g = j / parts;
    const bool inside = cut.start_of(g * parts) >= r0 &&
                        cut.start_of(min(cut.nsub, g * parts + parts)) <= r1;
    const bool mine_real = lane < count && (!inside || j == g * parts);
    const unsigned long long real = __ballot(mine_real);
    const int nreal = __popcll(real);
    // the slots that hold a partial, in order, as a list
    if (mine_real) lds_list[__popcll(real & ((1ull << lane) - 1ull))] = (uint8_t)lane;
    // (max, sum) of all these slots for the 16 head columns, the loads in flight
    // together: lane (column c, kg) fetches slot base + 4 * i + kg (unused slots
    // hold stale values that are never looked at; slots past the end repeat the last).
    // (Fetching them together with the accumulators of the first partials, one
    // round trip fewer on paper, measured 2 us slower at 8 short sequences.)
    const int c = min(lane & 15, a.group - 1);
    vfloat2 got[kSlots / 4];
#pragma unroll
    for (int i = 0; i < kSlots / 4; ++i) {
      const int s = min(base + 4 * i + (lane >> 4), expected - 1);
      got[i] = __builtin_bit_cast(vfloat2, __builtin_amdgcn_raw_buffer_load_b64(
                                               wm, (int)((s * rec_stride + c) * 8), 0, kDeviceScope));
    }
#pragma unroll
    for (int i = 0; i < kSlots / 4; ++i) lds_ml[(4 * i + (lane >> 4)) * 16 + (lane & 15)] = got[i];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (nreal > 0) {
      // the largest maximum among the real slots, per head: over the slots this
      // lane fetched, over the four lane rows, then from the head's column
      float m_chunk = kNegBig;
#pragma unroll
      for (int i = 0; i < kSlots / 4; ++i) {
        const int sl = min(4 * i + (lane >> 4), count - 1);
        if ((real >> sl) & 1ull) m_chunk = fmaxf(m_chunk, got[i].x);
      }
      m_chunk = fmaxf(m_chunk, __shfl_xor(m_chunk, 16, 64));
      m_chunk = fmaxf(m_chunk, __shfl_xor(m_chunk, 32, 64));
      m_chunk = __shfl(m_chunk, (lane & 48) | r, 64);
      const float m_new = fmaxf(m_run, m_chunk);
      const float keep = __builtin_amdgcn_exp2f((m_run - m_new) * a.scale_log2e);
      m_run = m_new;
      l_run *= keep;
#pragma unroll
      for (int jd = 0; jd < 8; ++jd) acc[jd] *= keep;
      for (int done = 0; done < nreal; done += 4 * lane_groups) {
        // four partials per lane group at a time; absent ones repeat the first
        // of the list with weight 0
        float w[4];
        vfloat4 v[4][8];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int n = done + k * lane_groups + lg;
          const bool have = n < nreal;
          const int idx = lds_list[have ? n : 0];
          const int off = (base + idx) * slot_bytes + lane_off;
#pragma unroll
          for (int i = 0; i < 8; ++i)
            v[k][i] = __builtin_bit_cast(
                vfloat4,
                __builtin_amdgcn_raw_buffer_load_b128(wo, off + i * piece_stride, 0, kDeviceScope));
          const vfloat2 ml = lds_ml[idx * 16 + r];
          w[k] = have ? __builtin_amdgcn_exp2f((ml.x - m_new) * a.scale_log2e) : 0.f;
          l_run = fmaf(w[k], ml.y, l_run);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            acc[0][e] = fmaf(w[k], v[k][2 * e].x, acc[0][e]);
            acc[1][e] = fmaf(w[k], v[k][2 * e].y, acc[1][e]);
            acc[2][e] = fmaf(w[k], v[k][2 * e].z, acc[2][e]);
            acc[3][e] = fmaf(w[k], v[k][2 * e].w, acc[3][e]);
            acc[4][e] = fmaf(w[k], v[k][2 * e + 1].x, acc[4][e]);
            acc[5][e] = fmaf(w[k], v[k][2 * e + 1].y, acc[5][e]);
            acc[6][e] = fmaf(w[k], v[k][2 * e + 1].z, acc[6][e]);
            acc[7][e] = fmaf(w[k], v[k][2 * e + 1].w, acc[7][e]);
          }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();   // the next pass overwrites lds_ml and the list
  }
  // the sum over the lane groups, into every lane
#define NVJ_ADD_LANE_GROUPS(N)                                         \
  if (gp <= N) {                                                       \
    l_run += row_rotate<N>(l_run);                                     \
    _Pragma("unroll") for (int jd = 0; jd < 8; ++jd)                   \
      _Pragma("unroll") for (int e = 0; e < 4; ++e)                    \
        acc[jd][e] += row_rotate<N>(acc[jd][e]);                       \
  }
  NVJ_ADD_LANE_GROUPS(8)
  NVJ_ADD_LANE_GROUPS(4)
  NVJ_ADD_LANE_GROUPS(2)
  NVJ_ADD_LANE_GROUPS(1)
#undef NVJ_ADD_LANE_GROUPS
  write_output<D, F16>(a, b, kvh, lane, acc, l_run);
}

// grid.x = num_wgs, block = 512.  `min_steps`: fewest steps a sub-run may have
// (in units of 1 << shift steps); `shift`: see Cut.
template <int D, bool F16, int VG = 0>
__global__ __launch_bounds__(512) void paged_decode_balanced_kernel(DecodeArgs a, int batch,
                                                                    int num_wgs, int min_steps,
                                                                    int hpw, int wr_hpw, int wr_hpw_alt,
                                                                    int wr_tol, int shift,
                                                                    int32_t* counters) {
  using H = HeadDim<D>;
  constexpr int NW = 8;
  __shared__ uint4 k_tile[NW][kStep * H::kLdsRowPieces];
  constexpr int kLanesWithDims = D / 32 * 16;   // lanes whose k-group holds real dims
  static_assert(sizeof(uint4) * kStep * H::kLdsRowPieces >= 34 * kLanesWithDims * sizeof(float),
                "a wave's K tile must hold its partial");
  // whole-row layout only: the lengths of the batch where any lane can index
  // them, the order the sequences are dealt to the workgroups in, and per wave
  // the partial of a piece that has to wait for the rest of its row
  __shared__ int wr_ctx[kKeptSequences];
  __shared__ int wr_steps[kKeptSequences];    // steps of every sequence
  __shared__ __align__(16) int wr_key[kKeptSequences];   // sorting keys
  __shared__ int wr_order[kKeptSequences];    // sequence of every rank by length
  __shared__ int wr_sorted[kKeptSequences];   // its steps
  __shared__ float wr_parked[NW][34 * kLanesWithDims];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int g = blockIdx.x;
  const int cap = a.max_blocks * a.block_size;

  auto ctx_of = [&](int idx) { return idx < batch ? min(max(a.context_lens[idx], 0), cap) : 0; };
  auto steps_of = [&](int idx) { return (ctx_of(idx) + kStep - 1) / kStep; };

  // One pass over the batch, 64 sequences at a time: total number of steps,
  // and for the first kKeep groups the per-lane (length, steps before) pairs
  // are kept so that locating a position below needs no second read.
  constexpr int kKeep = kKeptSequences / 64;
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
      total += __builtin_amdgcn_readlane(incl, 63);
    }
  }
  total_kept = total;
  for (int base = kKeep * 64; base < batch; base += 64) {
    const int n = steps_of(base + lane);
    total += __builtin_amdgcn_readlane(wave_inclusive_scan(n), 63);
  }
  // No step belongs to an empty sequence: its output row (zeros, 0 / (0 + 1e-9))
  // is written here, sequence b by workgroup b modulo the grid.  The lengths of
  // the first kKeep * 64 sequences are in registers already.
  for (int b = g; b < batch; b += gridDim.x) {
    int c;
    if (b < kKeep * 64) {
      int mine = kept_ctx[0];
#pragma unroll
      for (int k = 1; k < kKeep; ++k) mine = (b >> 6) == k ? kept_ctx[k] : mine;
      c = __shfl(mine, b & 63, 64);
    } else {
      c = min(as_constant(a.context_lens)[b], cap);
    }
    if (__builtin_amdgcn_readfirstlane(c) <= 0) {
      uint4* orow = a.out + (int64_t)b * a.num_heads * H::kPieces;
      for (int i = threadIdx.x; i < a.num_heads * H::kPieces; i += NW * 64)
        orow[i] = make_uint4(0u, 0u, 0u, 0u);
    }
  }

  // -------------------------------------------------------------------------
  // Whole-row layout.  When whole rows can be dealt to the workgroups so that
  // no workgroup gets more than (1 + wr_tol / 256) times its share of the
  // steps, no row is shared between workgroups: a row cut between the parts of
  // one workgroup is put together in LDS, and nothing goes through the
  // workspace or the counters.  The host offers it (wr_hpw > 0: the KV heads
  // per workgroup to use) when all lengths are among the kept ones and there
  // are at least as many rows as workgroups.  Rows are dealt in rounds of
  // num_wgs, forwards and backwards in turn (row of rank p goes to workgroup
  // p % num_wgs in an even round, num_wgs - 1 - p % num_wgs in an odd one),
  // first in the order of the batch - enough for lengths that are equal or
  // nearly so - and, when that is not balanced and there is more than one
  // round, by decreasing length, which pairs long rows with short ones.  Every
  // wave of the launch reads the same lengths and takes the same decision.
  // -------------------------------------------------------------------------
  if (wr_hpw > 0 && total > 0) {
    // every wave writes all the lengths and step counts itself (the same values
    // from each), so no wave has to wait for another before it reads them back
    int key[kKeep];
    int longest = 0, shortest = INT32_MAX;
#pragma unroll
    for (int k = 0; k < kKeep; ++k) {
      const bool real = k * 64 + lane < batch;
      const int n = (kept_ctx[k] + kStep - 1) / kStep;
      wr_ctx[k * 64 + lane] = real ? kept_ctx[k] : 0;
      wr_steps[k * 64 + lane] = real ? n : 0;
      // sorting key: more steps first, among equals the earlier sequence first;
      // unique, and below every real key for the padding behind the batch
      key[k] = real ? (n << 8) | (255 - (k * 64 + lane)) : -1 - (k * 64 + lane);
      longest = max(longest, real ? n : 0);
      shortest = min(shortest, real ? n : INT32_MAX);
    }
    longest = wave_max(longest);
    shortest = -wave_max(-shortest);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // Two candidates: wr_hpw KV heads per workgroup and, when whole rows of
    // that many heads cannot be dealt evenly enough, half as many (twice the
    // rows, another round or more to pair long with short; fewer heads side by
    // side stream a few percent slower, which is why it is second).
    int w_hpw = 0, w_rps = 1, rps_shift = 0, rows = 0, rounds = 0;
    bool whole_rows = false, sorted = false, ranked = false;
    for (int candidate = 0; candidate < 2 && !whole_rows; ++candidate) {
      w_hpw = candidate == 0 ? wr_hpw : wr_hpw_alt;
      if (w_hpw <= 0) break;
      w_rps = a.num_kv_heads / w_hpw;       // a power of two (the host sees to it)
      rps_shift = __builtin_ctz(w_rps);
      rows = batch * w_rps;
      rounds = (rows + num_wgs - 1) / num_wgs;
      // the largest number of steps any workgroup is dealt; steps_of_rank: the
      // steps of the sequence of a given rank (wr_steps in the order of the
      // batch, wr_sorted in the order by length)
      auto largest_deal = [&](const int* steps_of_rank) {
        int worst = 0;
        for (int w0 = 0; w0 < num_wgs; w0 += 64) {
          const int w = w0 + lane;
          int load = 0;
          for (int t = 0; t < rounds; ++t) {
            const int p = t * num_wgs + ((t & 1) ? num_wgs - 1 - w : w);
            if (w < num_wgs && p < rows) load += steps_of_rank[p >> rps_shift];
          }
          worst = max(worst, load);
        }
        return wave_max(worst);
      };
      const int64_t share = (int64_t)w_rps * total;   // num_wgs * a workgroup's share of the steps
      const auto fits = [&](int load, int tol) {
        return (int64_t)load * num_wgs * 256 <= share * (256 + tol);
      };
      // A row longer than the limit rules both orders out.  With one round
      // every workgroup gets one row and the longest row decides.  With more
      // rounds the order of the batch is only taken when it is as good as
      // balanced (and only looked at when the lengths are within an eighth of
      // each other); otherwise the order by length gets its chance.
      if (!fits(longest, wr_tol)) continue;
      sorted = false;
      if (rounds == 1) {
        whole_rows = true;
        break;
      }
      if ((longest - shortest) * 8 <= longest &&
          fits(largest_deal(wr_steps), min(wr_tol, kWholeRowTightTolerance))) {
        whole_rows = true;
        break;
      }
      if (!ranked) {
        // Rank of every sequence by decreasing key: two threads per sequence
        // count, over half of the batch each, the keys above its own.  The keys
        // go through LDS (every wave writes all of them, the same values from
        // each) and are read back four at a time, eight reads in flight.
#pragma unroll
        for (int k = 0; k < kKeep; ++k) wr_key[k * 64 + lane] = key[k];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int i = threadIdx.x >> 1, half = threadIdx.x & 1;
        const int mine = wr_key[i];
        const int quads = (batch + 3) / 4;            // int4 groups that hold real keys
        const int per_half = (quads + 1) / 2;
        int above = 0;
        for (int j0 = half * per_half; j0 < min(quads, (half + 1) * per_half); j0 += 8) {
          int4 k4[8];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            k4[u] = reinterpret_cast<const int4*>(wr_key)[min(j0 + u, kKeptSequences / 4 - 1)];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const bool in = j0 + u < min(quads, (half + 1) * per_half);
            above += (in && k4[u].x > mine ? 1 : 0) + (in && k4[u].y > mine ? 1 : 0) +
                     (in && k4[u].z > mine ? 1 : 0) + (in && k4[u].w > mine ? 1 : 0);
          }
        }
        above += __builtin_amdgcn_update_dpp(0, above, kDppQuadXor1, 0xF, 0xF, false);
        if (half == 0 && i < batch) {
          wr_order[above] = i;
          wr_sorted[above] = mine >> 8;
        }
        __syncthreads();
        ranked = true;
      }
      sorted = true;
      whole_rows = fits(largest_deal(wr_sorted), wr_tol);
    }
    if (whole_rows) {
      const int w_parts = NW / w_hpw;
      const int part = wave / w_hpw;
      const int h_in_row = wave - part * w_hpw;
      // the rows dealt to this workgroup, in the order of the rounds
      auto dealt_row = [&](int t, int& seq, int& hg, int& ctx) {
        const int p = t * num_wgs + ((t & 1) ? num_wgs - 1 - g : g);
        seq = 0; hg = 0; ctx = 0;
        if (p < rows) {
          const int rank = p / w_rps;
          seq = sorted ? wr_order[rank] : rank;
          hg = p - rank * w_rps;
          ctx = wr_ctx[seq];
        }
        seq = __builtin_amdgcn_readfirstlane(seq);
        hg = __builtin_amdgcn_readfirstlane(hg);
        ctx = __builtin_amdgcn_readfirstlane(max(ctx, 0));
      };
      int mine = 0;   // steps dealt to this workgroup
      for (int t = 0; t < rounds; ++t) {
        int seq, hg, ctx;
        dealt_row(t, seq, hg, ctx);
        mine += (ctx + kStep - 1) / kStep;
      }
      // the steps are cut into equal runs for the parts; a part's first piece,
      // when it does not start a row, waits in LDS for the part that does
      const int xs = (int)((int64_t)part * mine / w_parts);
      const int xe = (int)((int64_t)(part + 1) * mine / w_parts);
      f32x4 acc[8];
#pragma unroll
      for (int jd = 0; jd < 8; ++jd) acc[jd] = f32x4{0.f, 0.f, 0.f, 0.f};
      float m_run = kNegBig, l_run = 0.f;
      bool owes = false;       // acc holds the first piece of a row that goes on in later parts
      int owed_b = 0, owed_kvh = 0, owed_end = 0;
      const bool holds_dims = lane < kLanesWithDims;
      int row_start = 0;
      for (int t = 0; t < rounds && row_start < xe; ++t) {
        int seq, hg, ctx;
        dealt_row(t, seq, hg, ctx);
        const int nb = (ctx + kStep - 1) / kStep;
        const int lo = max(xs, row_start), hi = min(xe, row_start + nb);
        if (lo < hi) {
          const int st = lo - row_start, en = hi - row_start;
          const int kvh = hg * w_hpw + h_in_row;
          const int t0 = __builtin_amdgcn_readfirstlane(st * kStep);
          const int t1 = __builtin_amdgcn_readfirstlane(min(ctx, en * kStep));
          if constexpr (VG > 0)
            compute_segment_valu<VG>(a, k_tile[wave], seq, kvh, t0, t1, lane, acc, m_run, l_run);
          else if constexpr (VG < 0)
            compute_segment_loads_only(a, seq, kvh, t0, t1, lane, acc, m_run, l_run);
          else
            compute_segment<D, F16>(a, k_tile[wave], seq, kvh, t0, t1, lane, acc, m_run, l_run);
          if (st > 0) {
            // the row started in an earlier part: park the piece for it
            if (holds_dims) {
              float* slot = wr_parked[wave] + lane;
#pragma unroll
              for (int jd = 0; jd < 8; ++jd)
#pragma unroll
                for (int e = 0; e < 4; ++e) slot[(4 * jd + e) * kLanesWithDims] = acc[jd][e];
              slot[32 * kLanesWithDims] = m_run;
              slot[33 * kLanesWithDims] = l_run;
            }
          } else if (en == nb) {
            write_output<D, F16>(a, seq, kvh, lane, acc, l_run);
          } else {
            // the row goes on in the next part(s): this is the run's last segment
            owes = true; owed_b = seq; owed_kvh = kvh; owed_end = row_start + nb;
          }
        }
        row_start += nb;
      }
      __syncthreads();
      if (owes) {
        if (holds_dims) {
          for (int p = part + 1; p < w_parts; ++p) {
            const int ps = (int)((int64_t)p * mine / w_parts);
            const int pe = (int)((int64_t)(p + 1) * mine / w_parts);
            if (ps >= owed_end) break;
            if (pe > ps)
              add_partial_from_lds<kLanesWithDims>(wr_parked[p * w_hpw + h_in_row] + lane,
                                                   a.scale_log2e, acc, m_run, l_run);
          }
        }
        write_output<D, F16>(a, owed_b, owed_kvh, lane, acc, l_run);
      }
      return;
    }
  }
  const int parts = NW / hpw;
  const int rows_per_seq = a.num_kv_heads / hpw;
  const int part = wave / hpw;
  const int h_in_row = wave - part * hpw;
  Cut cut;
  cut.axis = rows_per_seq * total;
  cut.shift = shift;
  cut.units = (cut.axis + (1 << shift) - 1) >> shift;
  cut.nsub = max(1, min(num_wgs * parts, cut.units / min_steps));
  if (cut.axis == 0 || g * parts >= cut.nsub) return;
  const int nparts = min(parts, cut.nsub - g * parts);   // parts of this workgroup that have work
  const int start = cut.start_of(g * parts);
  const int end = cut.start_of(g * parts + nparts);

  // the sequence whose rows hold axis position x: its index, the steps before
  // it and its length (all wave-uniform)
  auto locate = [&](int x, int& b, int& before, int& ctx) {
    b = batch; before = total; ctx = 0;
    bool found = false;
#pragma unroll
    for (int k = 0; k < kKeep; ++k) {
      const int n = (kept_ctx[k] + kStep - 1) / kStep;
      const int lo = rows_per_seq * kept_excl[k];
      const unsigned long long hit =
          __ballot(!found && n > 0 && lo <= x && x < lo + rows_per_seq * n);
      if (hit != 0ull) {
        const int src = __builtin_ctzll(hit);
        b = k * 64 + src;
        before = __shfl(kept_excl[k], src, 64);
        ctx = __shfl(kept_ctx[k], src, 64);
        found = true;
      }
    }
    if (!found) {
      int running = total_kept;
      for (int base = kKeep * 64; base < batch; base += 64) {
        const int c = ctx_of(base + lane);
        const int n = (c + kStep - 1) / kStep;
        const int incl = wave_inclusive_scan(n);
        const int lo = rows_per_seq * (running + incl - n);
        const unsigned long long hit = __ballot(n > 0 && lo <= x && x < lo + rows_per_seq * n);
        if (hit != 0ull) {
          const int src = __builtin_ctzll(hit);
          b = base + src;
          before = __shfl(running + incl - n, src, 64);
          ctx = __shfl(c, src, 64);
          break;
        }
        running += __builtin_amdgcn_readlane(incl, 63);
      }
    }
    b = __builtin_amdgcn_readfirstlane(b);
    before = __builtin_amdgcn_readfirstlane(before);
    ctx = __builtin_amdgcn_readfirstlane(ctx);
  };

  int b0, before0, ctx0;
  locate(start, b0, before0, ctx0);
  if (b0 >= batch || ctx0 <= 0) return;   // cannot happen when the prefix sums are right
  const int nb0 = (ctx0 + kStep - 1) / kStep;
  const int hg0 = (start - rows_per_seq * before0) / nb0;
  const int row0 = rows_per_seq * before0 + hg0 * nb0;   // axis position of the row's step 0
  const int xs = part < nparts ? cut.start_of(g * parts + part) : end;
  const int xe = part < nparts ? cut.start_of(g * parts + part + 1) : end;
  const int64_t subrun = (int64_t)g * parts + part;
  // Does the whole run of the workgroup lie inside one row?  Then every wave has
  // at most one segment, and the parts of a head meet in LDS before anything is
  // written.  Otherwise every wave walks its own sub-run across the rows.
  const bool single = end <= row0 + nb0;
  if (!single && xs >= xe) return;

  int b = b0, before = before0, ctx = ctx0;
  if (!single && part > 0) locate(xs, b, before, ctx);
  // Every quantity of the walk is wave-uniform; readfirstlane says so, so that
  // lengths, page lookups and address arithmetic stay on the scalar unit.  The
  // guards (b inside the batch, x not before the sequence) cannot fire when
  // the prefix sums are right; they keep every index in range regardless.
  int x = xs;
  int owed = 0, owed_b[2] = {0, 0}, owed_kvh[2] = {0, 0}, owed_row[2] = {0, 0}, owed_nb[2] = {1, 1};
  for (;;) {
    // ---- the next segment of this wave's sub-run: row (sb, hg), steps [st, en) ----
    int sb = 0, hg = 0, nb = 1, row = 0, st = 0, en = 0;
    bool have = false;
    while (x < xe && b < batch) {
      sb = __builtin_amdgcn_readfirstlane(b);
      nb = (ctx + kStep - 1) / kStep;
      const int seq0 = rows_per_seq * before;
      if (x < seq0) break;
      if (nb == 0 || x >= seq0 + rows_per_seq * nb) {  // empty sequence, or this one is finished
        before += nb;
        b = sb + 1;
        ctx = b < batch ? __builtin_amdgcn_readfirstlane(
                              min(max(as_constant(a.context_lens)[b], 0), cap))
                        : 0;
        continue;
      }
      hg = (x - seq0) / nb;
      row = seq0 + hg * nb;
      st = x - row;
      en = min(nb, st + (xe - x));
      have = true;
      break;
    }
    if (!have && !single) break;
    const int kvh = (single ? hg0 : hg) * hpw + h_in_row;
    f32x4 acc[8];
#pragma unroll
    for (int jd = 0; jd < 8; ++jd) acc[jd] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = kNegBig, l_run = 0.f;
    if (have) {
      const int t0 = __builtin_amdgcn_readfirstlane(st * kStep);
      const int t1 = __builtin_amdgcn_readfirstlane(min(ctx, en * kStep));
      if constexpr (VG > 0)
        compute_segment_valu<VG>(a, k_tile[wave], sb, kvh, t0, t1, lane, acc, m_run, l_run);
      else if constexpr (VG < 0)
        compute_segment_loads_only(a, sb, kvh, t0, t1, lane, acc, m_run, l_run);
      else
        compute_segment<D, F16>(a, k_tile[wave], sb, kvh, t0, t1, lane, acc, m_run, l_run);
      x += en - st;
    }

    bool direct = st == 0 && en == nb;   // the segment is the whole row
    int covers = 1;                      // sub-runs this wave's partial stands for
    if (single) {
      sb = b0; hg = hg0; nb = nb0; row = row0;
      direct = start == row0 && end == row0 + nb0;
      covers = nparts;
      if (nparts > 1) {
        const bool holds_dims = lane < kLanesWithDims;
        if (part > 0 && have) {
          // value v of lane l at float v * kLanesWithDims + l of the wave's own tile
          if (holds_dims) {
            float* mine = reinterpret_cast<float*>(k_tile[wave]) + lane;
#pragma unroll
            for (int jd = 0; jd < 8; ++jd)
#pragma unroll
              for (int e = 0; e < 4; ++e) mine[(4 * jd + e) * kLanesWithDims] = acc[jd][e];
            mine[32 * kLanesWithDims] = m_run;
            mine[33 * kLanesWithDims] = l_run;
          }
        }
        __syncthreads();
        if (part > 0) return;
        if (holds_dims) {
          for (int p = 1; p < nparts; ++p) {
            add_partial_from_lds<kLanesWithDims>(
                reinterpret_cast<const float*>(k_tile[wave + p * hpw]) + lane, a.scale_log2e, acc,
                m_run, l_run);
          }
        }
      }
      if (part > 0) return;
    }

    if (direct) {
      write_output<D, F16>(a, sb, kvh, lane, acc, l_run);
    } else {
      const int64_t slot = subrun + (int64_t)sb * rows_per_seq + hg;
      write_partial_coherent<D>(a, balanced_record(a, slot, hpw, h_in_row), lane, acc, m_run,
                                l_run);
      if (arrive(a, counters, sb, kvh, row, row + nb, cut, covers, lane)) {
        // at most the first and the last segment of a sub-run are not whole rows
        if (owed == 0) { owed_b[0] = sb; owed_kvh[0] = kvh; owed_row[0] = row; owed_nb[0] = nb; }
        else { owed_b[1] = sb; owed_kvh[1] = kvh; owed_row[1] = row; owed_nb[1] = nb; }
        ++owed;
      }
    }
    if (single) break;
  }
  // the merges this wave owes, after its own work
  for (int i = 0; i < owed; ++i) {
    const int ob = __builtin_amdgcn_readfirstlane(i == 0 ? owed_b[0] : owed_b[1]);
    const int okvh = __builtin_amdgcn_readfirstlane(i == 0 ? owed_kvh[0] : owed_kvh[1]);
    const int orow = __builtin_amdgcn_readfirstlane(i == 0 ? owed_row[0] : owed_row[1]);
    const int onb = __builtin_amdgcn_readfirstlane(i == 0 ? owed_nb[0] : owed_nb[1]);
    merge_row<D, F16>(a, k_tile[wave], ob, okvh, hpw, orow, orow + onb, cut, lane);
  }
}

// Sets n int32 to zero (the counters of the balanced split; a kernel, not a
// memset, so that the launch can be recorded into a graph).
__global__ __launch_bounds__(256) void zero_int32_kernel(int32_t* p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}

// Second pass of the fixed split: merge the partials of one (sequence, query
// head).  grid = (B, Hq), block = head_dim lanes, one per output dim.  The
// partials of sequence b are slots b*max_chunks .. + ceil(ctx/chunk).  A
// sequence with one partial was written by the split kernel itself; an empty
// one gives zeros.
__global__ __launch_bounds__(kMaxHeadDim) void paged_decode_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const int32_t* __restrict__ context_lens, uint16_t* __restrict__ out, int num_heads, int chunk,
    int max_chunks, int max_positions, float scale_log2e, bool f16) {
  const int b = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
  const int head_dim = blockDim.x;
  const int ctx = min(context_lens[b], max_positions);
  const int nparts = ctx <= 0 ? 0 : (ctx + chunk - 1) / chunk;
  const int64_t first = (int64_t)b * max_chunks;
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

// Compute units of the current device (256 on an MI355X), looked up once per
// device; 256 when no device can be asked (argument checks without a GPU).
int compute_units() {
  constexpr int kMaxDevicesSeen = 64;
  static std::atomic<int> cached[kMaxDevicesSeen];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevicesSeen) {
    (void)hipGetLastError();   // not an error of any launch
    return 256;
  }
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      n <= 0) {
    (void)hipGetLastError();
    return 256;
  }
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

// KV heads per 8-wave workgroup of the whole-sequence mode: as many as still
// give one (sequence, head group) row per CU, so that a sequence is split over
// the waves of a workgroup no finer than needed; it must divide the number of
// KV heads.
int heads_per_workgroup(int64_t batch, int num_kv_heads) {
  const int cus = compute_units();
  int hpw = 8;
  while (hpw > 1 && (num_kv_heads % hpw != 0 || batch * (num_kv_heads / hpw) < cus)) hpw /= 2;
  return hpw;
}

// KV heads per 8-wave workgroup of the balanced split.  Two forces pull apart.
// The heads of one workgroup read adjacent pieces of every position's row, and
// a stream-bound launch runs faster with more of them side by side: 32
// sequences of 16k..32k positions take 506 / 471 / 457 / 460 us with 1 / 2 / 4
// / 8 heads of 128 per workgroup (head_dim 64 ranks the same way).  Against
// that, the partials one wave has to merge per (sequence, head) grow with the
// heads per workgroup, because the sub-runs are then spread over fewer rows: a
// single sequence of 32k positions takes 38 / 45 / 67 / 109 us.  The rule below
// is the best or within 3 % of it over batch 1..256 x 512..32768 positions x
// 2, 4, 8 KV heads, ragged and uniform lengths: 4 heads from batch 32 up, or
// from batch 16 when the table spans 4096 positions; 1 head for up to 16
// (sequence, head) pairs when the table spans 6144 positions or more; else 2.
int balanced_heads_per_workgroup(int64_t batch, int num_kv_heads, int64_t max_steps) {
  int hpw = 2;
  if (batch * num_kv_heads <= 16 && max_steps >= 192) hpw = 1;
  else if (batch >= 32 || (batch >= 16 && max_steps >= 128)) hpw = 4;
  while (hpw > 1 && num_kv_heads % hpw != 0) hpw /= 2;
  return hpw;
}

// Balanced mode launches at most one workgroup per CU, and never gives a wave
// fewer than this many 32-position steps.
constexpr int kMinBalancedSteps = 1;

// Whole rows are dealt to the workgroups when no workgroup gets more than
// 1 + kWholeRowTolerance / 256 times the mean number of steps.  The launch is
// bound by the memory system as a whole, not by its slowest workgroup: while
// workgroups with less to do finish, the others stream faster, so an uneven
// deal costs far less than its unevenness.  Measured against the equal cut with
// shared rows (256 sequences, 2 rows each, lengths log-uniform or uniform):
// 9 % unevenness 195 against 213 us, 16 % 174 against 187, 34 % 148 against
// 149, 56 % 250 against 231; one row per workgroup (64 sequences around 3500
// positions): 9 % 153 against 165, 15 % 146 against 154, 25 % 137 against 142.
constexpr int kWholeRowTolerance = 64;

// Waves per workgroup of the fixed split = KV heads a workgroup covers: the
// largest of 8, 4, 2, 1 that divides the number of KV heads.
int waves_per_workgroup(int num_kv_heads) {
  return num_kv_heads % 8 == 0 ? 8 : num_kv_heads % 4 == 0 ? 4 : num_kv_heads % 2 == 0 ? 2 : 1;
}

// The counter region of the balanced split: word 0 is the stale flag, then one
// int32 per (sequence, KV head as the kernels walk them); padded to 256 bytes.
size_t counter_region_bytes(int64_t batch, int64_t kv_heads) {
  return ((size_t)(batch * kv_heads + 1) * sizeof(int32_t) + 255) / 256 * 256;
}

// Workspace layout.  Fixed chunks: partials of batch * max_chunks slots, every
// slot holding all query heads.  Balanced: first the counters, one int32 per
// (sequence, KV head), padded to 256 bytes; then the partials of slots =
// sub-runs + rows, a slot holding the query heads of hpw KV heads.
struct WorkspacePlan {
  int64_t records;  // partial records (one query head each)
  int max_chunks;   // fixed-chunk mode only
  int num_wgs, hpw, wr_hpw, wr_hpw_alt, shift;  // balanced mode only
  size_t counter_bytes;
  size_t bytes;
};

bool plan_workspace(int64_t batch, int64_t num_heads, int64_t head_dim, int64_t max_blocks,
                    int64_t block_size, int num_kv_heads, int chunk, WorkspacePlan* plan) {
  if (chunk == 0) {
    const int64_t max_steps = (max_blocks * block_size + kStep - 1) / kStep;
    const int hpw = balanced_heads_per_workgroup(batch, num_kv_heads, max_steps);
    const int parts = 8 / hpw;
    const int64_t rows_per_seq = num_kv_heads / hpw;
    const int64_t axis = rows_per_seq * batch * max_steps;
    if (axis > INT32_MAX / 2) return false;
    int64_t wgs = (axis + (int64_t)parts * kMinBalancedSteps - 1) / (parts * kMinBalancedSteps);
    const int64_t cus = compute_units();
    wgs = wgs < 1 ? 1 : wgs > cus ? cus : wgs;
    plan->num_wgs = (int)wgs;
    plan->hpw = hpw;
    // (units + 1) * sub-runs must fit 31 bits (Cut): coarser units for a very long axis
    plan->shift = 0;
    while ((((axis >> plan->shift) + 2) * wgs * parts) >> 31) ++plan->shift;
    // The whole-row layout of the kernel (no partials at all) is offered when the
    // kernel keeps every length in registers and there is a row for every
    // workgroup: with as many heads per workgroup as still give that, 2 at least
    // (rows of 1 head are only worth it as the second choice: 32 equal sequences
    // of 8192 positions take 167 us that way against 164 with the equal cut), and
    // as a second choice with half as many heads, which gives the kernel another
    // round or more of rows to pair long ones with short ones (64 sequences of
    // 2048..6144 positions: 175 us with 1 head per workgroup, by length, against
    // 180 with the equal cut; 128 of 2000..6000: 321 with 2 heads against 329).
    // The layout needs no workspace of its own.
    plan->wr_hpw = plan->wr_hpw_alt = 0;
    const auto whole_rows_can_use = [&](int h) {
      const int rps = h > 0 && num_kv_heads % h == 0 ? num_kv_heads / h : 0;
      return rps > 0 && (rps & (rps - 1)) == 0 &&   // the kernel divides by shifting
             batch * rps >= wgs;
    };
    if (batch <= kKeptSequences && wgs <= kMaxWholeRowWorkgroups)
      for (int h = hpw; h >= 2; h /= 2)
        if (num_kv_heads % h == 0 && batch * (num_kv_heads / h) >= wgs) {
          if (whole_rows_can_use(h)) {
            plan->wr_hpw = h;
            if (whole_rows_can_use(h / 2)) plan->wr_hpw_alt = h / 2;
          }
          break;
        }
    plan->max_chunks = 0;
    const int64_t slots = wgs * parts + batch * rows_per_seq;
    plan->records = slots * hpw * (num_heads / num_kv_heads);
    plan->counter_bytes = counter_region_bytes(batch, num_kv_heads);
    plan->bytes = plan->counter_bytes + (size_t)plan->records * (head_dim + 2) * sizeof(float);
    return true;
  }
  const int64_t mc = (max_blocks * block_size + chunk - 1) / chunk;
  if (batch * mc > INT32_MAX) return false;
  plan->num_wgs = plan->hpw = plan->wr_hpw = plan->wr_hpw_alt = plan->shift = 0;
  plan->max_chunks = (int)mc;
  plan->records = batch * mc * num_heads;
  plan->counter_bytes = 0;
  plan->bytes = (size_t)plan->records * (head_dim + 2) * sizeof(float);
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
  return batch * ((int)heads / heads_per_workgroup(batch, (int)heads));
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

namespace {
// The launch behind every decode entry point.  `ext_counters` != NULL: the
// counters of the balanced split live there and `workspace` holds the partials
// only (no counter header in front of them).
int launch_decode(void* stream, const void* q, const void* k_cache, const void* v_cache,
                  const int32_t* block_tables, const int32_t* context_lens, void* out,
                  void* workspace, size_t workspace_bytes, int32_t* ext_counters, int32_t batch,
                  int32_t num_heads, int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                  int32_t max_blocks, int32_t num_blocks, float scale, int32_t chunk,
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
    return NVJ_ERR_ALIGNMENT;
  // the vector-ALU measurement variant exists for one shape family only
  const bool valu = (phases & NVJ_PHASE_VALU_PRODUCTS) != 0;
  if (valu && (head_dim != 128 || f16 || kv_rep != 1 || (group != 4 && group != 8) ||
               num_kv_heads % 8 != 0 || chunk > 0))
    return NVJ_ERR_UNSUPPORTED;
  // the loads-only measurement variant: head_dim 128, bf16, not with a fixed chunk
  const bool loads_only = (phases & NVJ_PHASE_LOADS_ONLY) != 0;
  if (loads_only && (valu || head_dim != 128 || f16 || chunk > 0)) return NVJ_ERR_UNSUPPORTED;
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
    const int hpw = heads_per_workgroup(batch, num_kv_heads);
    const dim3 grid((unsigned)(batch * (num_kv_heads / hpw))), block(512);
    hipError_t rc;
    if (loads_only) rc = nvj::launch(paged_decode_whole_kernel<8, 128, false, -1>, grid, block, s, a, hpw);
    else if (valu && group == 4) rc = nvj::launch(paged_decode_whole_kernel<8, 128, false, 4>, grid, block, s, a, hpw);
    else if (valu) rc = nvj::launch(paged_decode_whole_kernel<8, 128, false, 8>, grid, block, s, a, hpw);
    else if (head_dim == 128 && !f16) rc = nvj::launch(paged_decode_whole_kernel<8, 128, false>, grid, block, s, a, hpw);
    else if (head_dim == 128) rc = nvj::launch(paged_decode_whole_kernel<8, 128, true>, grid, block, s, a, hpw);
    else if (!f16) rc = nvj::launch(paged_decode_whole_kernel<8, 64, false>, grid, block, s, a, hpw);
    else rc = nvj::launch(paged_decode_whole_kernel<8, 64, true>, grid, block, s, a, hpw);
    return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
  }

  WorkspacePlan plan = {0, 1, 0, 0, 0, 0, 0, 0, 0};
  if (max_blocks > 0) {
    if (!plan_workspace(batch, num_heads, head_dim, max_blocks, block_size, num_kv_heads, chunk,
                        &plan))
      return NVJ_ERR_BAD_SHAPE;
    const size_t header = ext_counters ? 0 : plan.counter_bytes;
    if (!workspace || workspace_bytes < plan.bytes - plan.counter_bytes + header)
      return NVJ_ERR_WORKSPACE;
    int32_t* counters = ext_counters ? ext_counters : static_cast<int32_t*>(workspace);
    a.part_o = reinterpret_cast<float*>(static_cast<char*>(workspace) + header);
    a.part_ml = a.part_o + plan.records * head_dim;

    if (chunk == 0) {
      // one launch: the workgroup that completes a sequence merges it
      if (phases & NVJ_PHASE_CLEAR_COUNTERS) {
        const int n = (int)(plan.counter_bytes / sizeof(int32_t));   // stale flag, counters, padding
        if (nvj::launch(zero_int32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), s,
                        counters, n) != hipSuccess)
          return NVJ_ERR_LAUNCH;
      }
      if (!(phases & NVJ_PHASE_SPLITK)) return NVJ_OK;
      const dim3 grid((unsigned)plan.num_wgs);
      hipError_t rc;
#define NVJ_LAUNCH_BALANCED(DV, F16V, VGV)                                                     \
  rc = nvj::launch(paged_decode_balanced_kernel<DV, F16V, VGV>, grid, dim3(512), s, a, batch, \
                   plan.num_wgs, kMinBalancedSteps, plan.hpw,                      \
                   (phases & NVJ_PHASE_SHARED_ROWS) ? 0 : plan.wr_hpw, plan.wr_hpw_alt,       \
                   kWholeRowTolerance, plan.shift, counters)
      if (loads_only) NVJ_LAUNCH_BALANCED(128, false, -1);
      else if (valu && group == 4) NVJ_LAUNCH_BALANCED(128, false, 4);
      else if (valu) NVJ_LAUNCH_BALANCED(128, false, 8);
      else if (head_dim == 128 && !f16) NVJ_LAUNCH_BALANCED(128, false, 0);
      else if (head_dim == 128) NVJ_LAUNCH_BALANCED(128, true, 0);
      else if (!f16) NVJ_LAUNCH_BALANCED(64, false, 0);
      else NVJ_LAUNCH_BALANCED(64, true, 0);
#undef NVJ_LAUNCH_BALANCED
      return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
    }

    if (phases & NVJ_PHASE_SPLITK) {
      const int nw = waves_per_workgroup(num_kv_heads);
      const dim3 grid((unsigned)(batch * plan.max_chunks), (unsigned)(num_kv_heads / nw));
      // one instantiation per (waves per workgroup, head_dim, element type)
      hipError_t rc;
#define NVJ_LAUNCH_FIXED(NWV, DV)                                                              \
  rc = f16 ? nvj::launch(paged_decode_splitk_kernel<NWV, DV, true>, grid, dim3(NWV * 64), s, a, \
                         chunk, plan.max_chunks)                                               \
           : nvj::launch(paged_decode_splitk_kernel<NWV, DV, false>, grid, dim3(NWV * 64), s, a, \
                         chunk, plan.max_chunks)
      switch (nw * 1000 + head_dim) {
        case 8128: NVJ_LAUNCH_FIXED(8, 128); break;
        case 4128: NVJ_LAUNCH_FIXED(4, 128); break;
        case 2128: NVJ_LAUNCH_FIXED(2, 128); break;
        case 1128: NVJ_LAUNCH_FIXED(1, 128); break;
        case 8064: NVJ_LAUNCH_FIXED(8, 64); break;
        case 4064: NVJ_LAUNCH_FIXED(4, 64); break;
        case 2064: NVJ_LAUNCH_FIXED(2, 64); break;
        default: NVJ_LAUNCH_FIXED(1, 64); break;
      }
#undef NVJ_LAUNCH_FIXED
      if (rc != hipSuccess) return NVJ_ERR_LAUNCH;
    }
  } else {
    chunk = kStep;  // no pages at all: every sequence is empty, the second pass writes zeros
  }
  if (!(phases & NVJ_PHASE_COMBINE)) return NVJ_OK;
  const hipError_t rc = nvj::launch(
      paged_decode_combine_kernel, dim3((unsigned)batch, (unsigned)num_heads), dim3(head_dim), s,
      a.part_o, a.part_ml, context_lens, static_cast<uint16_t*>(out), num_heads, chunk,
      plan.max_chunks, max_blocks * block_size, a.scale_log2e, f16);
  return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

}  // namespace

extern "C" int nvj_paged_decode_launch_phases(void* stream, const void* q, const void* k_cache,
                                              const void* v_cache, const int32_t* block_tables,
                                              const int32_t* context_lens, void* out,
                                              void* workspace, size_t workspace_bytes,
                                              int32_t batch, int32_t num_heads,
                                              int32_t num_kv_heads, int32_t head_dim,
                                              int32_t block_size, int32_t max_blocks,
                                              int32_t num_blocks, float scale, int32_t chunk,
                                              int32_t dtype, uint32_t phases) {
  return launch_decode(stream, q, k_cache, v_cache, block_tables, context_lens, out, workspace,
                       workspace_bytes, nullptr, batch, num_heads, num_kv_heads, head_dim,
                       block_size, max_blocks, num_blocks, scale, chunk, dtype, phases);
}

extern "C" size_t nvj_paged_decode_counter_bytes(int32_t batch, int32_t num_heads,
                                                 int32_t num_kv_heads) {
  if (batch <= 0 || num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0) return 0;
  const size_t heads =
      (size_t)num_kv_heads * virtual_heads_per_cache_head(num_heads / num_kv_heads);
  return counter_region_bytes(batch, (int64_t)heads);
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
                                        NVJ_PHASE_SPLITK | NVJ_PHASE_COMBINE |
                                            NVJ_PHASE_CLEAR_COUNTERS);
}

// ---------------------------------------------------------------------------
// The library's own device array.  Its first kCounterRegion bytes are a counter
// region of the balanced split that belongs to no caller (the same words
// whatever the shape of a call: zero when the library is loaded, put back to
// zero by every launch); the rest is the workspace of the entry point that
// allocates nothing.  The array's name is a host-side stand-in; its device
// address is looked up once per device (hipGetSymbolAddress) and only that
// address is ever handed to a kernel.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[NVJ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
constexpr size_t kCounterRegion = 64u << 10;
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

extern "C" int nvj_paged_decode_library_counters(void** counters, size_t* bytes) {
  if (!counters) return NVJ_ERR_NULL_POINTER;
  if (bytes) *bytes = kCounterRegion;
  return static_scratch_of_current_device(counters);
}

extern "C" int nvj_paged_decode_counters_reset(void* stream, void* counters,
                                               size_t counter_bytes) {
  if (!counters) {
    const int rc = static_scratch_of_current_device(&counters);
    if (rc != NVJ_OK) return rc;
    counter_bytes = kCounterRegion;
  }
  if (reinterpret_cast<uintptr_t>(counters) & 3u) return NVJ_ERR_ALIGNMENT;
  if (counter_bytes / sizeof(int32_t) > (size_t)INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  const int n = (int)(counter_bytes / sizeof(int32_t));
  if (n == 0) return NVJ_OK;
  return nvj::launch(zero_int32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256),
                     static_cast<hipStream_t>(stream), static_cast<int32_t*>(counters),
                     n) == hipSuccess
             ? NVJ_OK
             : NVJ_ERR_LAUNCH;
}

extern "C" int nvj_paged_decode_launch_counters(void* stream, const void* q, const void* k_cache,
                                                const void* v_cache, const int32_t* block_tables,
                                                const int32_t* context_lens, void* out,
                                                void* partials, size_t partial_bytes,
                                                void* counters, size_t counter_bytes,
                                                int32_t batch, int32_t num_heads,
                                                int32_t num_kv_heads, int32_t head_dim,
                                                int32_t block_size, int32_t max_blocks,
                                                int32_t num_blocks, float scale, int32_t dtype,
                                                uint32_t phases) {
  if (batch > 0 && max_blocks > 0) {
    const size_t need = nvj_paged_decode_counter_bytes(batch, num_heads, num_kv_heads);
    if (!counters) {
      // need == 0: invalid arguments, which the launch below reports by name
      if (need > kCounterRegion) return NVJ_ERR_SCRATCH_LIMIT;
      if (need > 0) {
        const int rc = static_scratch_of_current_device(&counters);
        if (rc != NVJ_OK) return rc;
      }
    } else {
      if (reinterpret_cast<uintptr_t>(counters) & 3u) return NVJ_ERR_ALIGNMENT;
      if (need > 0 && counter_bytes < need) return NVJ_ERR_WORKSPACE;
    }
  }
  return launch_decode(stream, q, k_cache, v_cache, block_tables, context_lens, out, partials,
                       partial_bytes, static_cast<int32_t*>(counters), batch, num_heads,
                       num_kv_heads, head_dim, block_size, max_blocks, num_blocks, scale, 0, dtype,
                       phases);
}

extern "C" int nvj_paged_decode_static_launch(void* stream, const void* q, const void* k_cache,
                                              const void* v_cache, const int32_t* block_tables,
                                              const int32_t* context_lens, void* out,
                                              int32_t batch, int32_t num_heads,
                                              int32_t num_kv_heads, int32_t head_dim,
                                              int32_t block_size, int32_t max_blocks,
                                              int32_t num_blocks, float scale, int32_t dtype) {
  void* base = nullptr;
  if (batch > 0 && max_blocks > 0) {
    const size_t need = nvj_paged_decode_workspace_bytes(batch, num_heads, head_dim, max_blocks,
                                                         block_size, num_kv_heads, 0);
    const size_t counters = nvj_paged_decode_counter_bytes(batch, num_heads, num_kv_heads);
    // need == 0: invalid arguments, which the launch below reports by name
    if (need > 0 && (counters > kCounterRegion ||
                     need - counters > NVJ_STATIC_SCRATCH_BYTES - kCounterRegion))
      return NVJ_ERR_SCRATCH_LIMIT;
    if (need > 0) {
      const int rc = static_scratch_of_current_device(&base);
      if (rc != NVJ_OK) return rc;
    }
  }
  char* partials = base ? static_cast<char*>(base) + kCounterRegion : nullptr;
  return launch_decode(stream, q, k_cache, v_cache, block_tables, context_lens, out, partials,
                       base ? (size_t)NVJ_STATIC_SCRATCH_BYTES - kCounterRegion : 0,
                       static_cast<int32_t*>(base), batch, num_heads, num_kv_heads, head_dim,
                       block_size, max_blocks, num_blocks, scale, 0, dtype,
                       NVJ_PHASE_SPLITK | NVJ_PHASE_COMBINE);
}

extern "C" const char* nvj_error_string(int code) {
  switch (code) {
    case NVJ_OK: return "ok";
    case NVJ_ERR_NULL_POINTER: return "a required pointer is NULL";
    case NVJ_ERR_BAD_SHAPE: return "invalid shape or size argument";
    case NVJ_ERR_UNSUPPORTED: return "unsupported head_dim / group size / block size / chunk";
    case NVJ_ERR_WORKSPACE: return "workspace missing or too small";
    case NVJ_ERR_ALIGNMENT: return "a pointer is not 16-byte aligned";
    case NVJ_ERR_LAUNCH: return "kernel launch failed";
    case NVJ_ERR_BAD_DTYPE: return "unknown element type code";
    case NVJ_ERR_SCRATCH_LIMIT:
      return "problem needs more than the library's static scratch (NVJ_STATIC_SCRATCH_BYTES)";
    default: return "unknown error code";
  }
}

extern "C" int nvj_abi_version(void) { return NVJ_ABI_VERSION; }

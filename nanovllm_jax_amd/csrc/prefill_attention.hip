// Variable-length causal prefill attention for gfx950 (CDNA4, wave64).
//
// Stands in for variable_length_attention_prefill (layers/attention.py:135-279
// of the reference) as called from Attention._prefill_attention (:331-364): q,
// k, v are the packed rows of the prompts being prefilled, sequence i owning q
// rows [cu_q[i], cu_q[i+1]) and k/v rows [cu_k[i], cu_k[i+1]).  Query position
// p of a sequence attends key positions <= p of the same sequence (the
// reference's mask `q_pos >= k_pos`, both counted from the start of the
// sequence, :232-243).  GQA maps query head h to kv head h / G.  Nothing is
// padded and nothing of size max_len^2 is materialised.
//
// MFMA-bound.  One workgroup = 4 waves = 128 query rows of one (sequence, query
// head); a wave owns 32 rows as two groups of 16 MFMA columns.  Keys are walked
// 32 at a time; the K tile and the V tile of a step are fetched once per
// workgroup and staged in LDS (double-buffered, one barrier per step):
//   * K as rows of 16-byte pieces (padded), read back as the A operand of
//     S^T[key, q] = K . Q^T  (v_mfma_f32_16x16x32_bf16, Q^T of both groups in
//     registers for the whole tile);
//   * V already transposed into A operands of O^T[dim, q] += V^T . P^T: the
//     loading lane holds 2 keys x 8 dims and writes, per dim, the 2-key pair
//     where the operand of (dim group, key group) expects it.
// Softmax is the fp32 online form on the accumulator layout; P^T comes out of
// the S^T accumulators already in B-operand layout (same reduction-slot <-> key
// map as the decode kernel).  Only tiles that touch the diagonal are masked.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nvj_paged_attn.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kD = 128;
constexpr int kPieces = 16;          // 16-byte pieces per (position, head) row
constexpr int kBM = 128;             // query rows per workgroup
constexpr int kWaves = 4;
constexpr int kRowsPerWave = kBM / kWaves;   // 32 = two column groups of 16
constexpr int kKeys = 32;            // keys per step
constexpr int kKRow = kPieces + 1;   // padded K row in LDS, in pieces
constexpr float kNegBig = -1.0e30f;
constexpr float kLazyLog2 = 8.0f;    // running max moves only for gains above 2^8
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  bf16x2 p = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, p);
}

typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;

// reduction slot j of key group kg stands for this key of the 32-key step
__device__ __forceinline__ int slot_key(int kg, int j) {
  return j < 4 ? 4 * kg + j : 16 + 4 * kg + (j - 4);
}

// Cooperative tile loads of a workgroup: K 2 pieces per thread, V 2 keys per
// thread.  K item i of the 512 (key, piece) pairs of a step: key = i / 16,
// piece = i % 16.  V: wave = key group, lane = (slot pair qd, piece r): the two
// keys of reduction slots 2*qd and 2*qd + 1 of that key group.  Keys are clamped to the last visible one, so nothing at or beyond
// k_end is read.
struct TileLoader {
  const char* k_head;   // first key row of the sequence for this kv head
  const char* v_head;
  uint32_t row_bytes;   // bytes between consecutive keys
  int last_key, tid, wave, r, qd;

  // One uniform 64-bit base per tile (its first key row) plus one 32-bit lane
  // offset per load; the last tile clamps every key to last_key.  Keys of a
  // tile are < 32 and row_bytes < 2^24 (checked by the host): 24-bit multiplies.
  __device__ __forceinline__ void issue_k(int step, uint4& k0, uint4& k1) const {
    const int ks = step * kKeys;
    const uint32_t piece_bytes = (uint32_t)(tid % kPieces) * 16u;
    int a0 = tid / kPieces, a1 = tid / kPieces + 16;   // items tid and tid + 256
    if (ks + kKeys - 1 > last_key) {
      const int cap = last_key - ks;   // >= 0: the tile starts at a visible key
      a0 = min(a0, cap);
      a1 = min(a1, cap);
    }
    const char* kb = k_head + (size_t)ks * row_bytes;
    k0 = *reinterpret_cast<const uint4*>(kb + (__umul24(a0, row_bytes) + piece_bytes));
    k1 = *reinterpret_cast<const uint4*>(kb + (__umul24(a1, row_bytes) + piece_bytes));
  }

  __device__ __forceinline__ void issue_v(int step, uint4& v0, uint4& v1) const {
    const int ks = step * kKeys;
    int b0 = slot_key(wave, 2 * qd), b1 = slot_key(wave, 2 * qd + 1);
    if (ks + kKeys - 1 > last_key) {
      const int cap = last_key - ks;
      b0 = min(b0, cap);
      b1 = min(b1, cap);
    }
    const char* vb = v_head + (size_t)ks * row_bytes;
    v0 = *reinterpret_cast<const uint4*>(vb + (__umul24(b0, row_bytes) + (uint32_t)r * 16u));
    v1 = *reinterpret_cast<const uint4*>(vb + (__umul24(b1, row_bytes) + (uint32_t)r * 16u));
  }

  __device__ __forceinline__ void stage_k(uint4* k_tile, const uint4& k0, const uint4& k1) const {
    const int piece = tid % kPieces, key = tid / kPieces;
    k_tile[key * kKRow + piece] = k0;
    k_tile[(key + 16) * kKRow + piece] = k1;
  }

  // 2 keys x 8 dims -> per dim the (key0, key1) pair, at slot pair 2*qd of the
  // operand of (dim jd, key group = wave, piece r)
  __device__ __forceinline__ void stage_v(uint4* vt_tile, const uint4& v0, const uint4& v1) const {
    uint32_t* vt32 = reinterpret_cast<uint32_t*>(vt_tile);
    const int base = (wave * kPieces + r) * 4 + qd;
    const int dim_stride = 4 * kPieces * 4;   // dwords between consecutive jd
    vt32[base + 0 * dim_stride] = __builtin_amdgcn_perm(v1.x, v0.x, 0x05040100u);
    vt32[base + 1 * dim_stride] = __builtin_amdgcn_perm(v1.x, v0.x, 0x07060302u);
    vt32[base + 2 * dim_stride] = __builtin_amdgcn_perm(v1.y, v0.y, 0x05040100u);
    vt32[base + 3 * dim_stride] = __builtin_amdgcn_perm(v1.y, v0.y, 0x07060302u);
    vt32[base + 4 * dim_stride] = __builtin_amdgcn_perm(v1.z, v0.z, 0x05040100u);
    vt32[base + 5 * dim_stride] = __builtin_amdgcn_perm(v1.z, v0.z, 0x07060302u);
    vt32[base + 6 * dim_stride] = __builtin_amdgcn_perm(v1.w, v0.w, 0x05040100u);
    vt32[base + 7 * dim_stride] = __builtin_amdgcn_perm(v1.w, v0.w, 0x07060302u);
  }
};

// NaN-propagating maximum: one v_maximum3_f32 per three values, no
// canonicalising moves on MFMA results.
__device__ __forceinline__ float max2(float a, float b) {
  return __builtin_elementwise_maximum(a, b);
}
__device__ __forceinline__ float max_of8(const f32x4& a, const f32x4& b) {
  const float t1 = max2(max2(a[0], a[1]), a[2]);
  const float t2 = max2(max2(a[3], b[0]), b[1]);
  return max2(max2(max2(b[2], b[3]), t1), t2);
}

// S^T of one 32-key tile against both column groups (16 query rows each):
// sc[g][h] holds keys 16*h + 4*kg + e of the tile for query row r of group g.
__device__ __forceinline__ void scores_of_tile(const uint4* kt, const bf16x8 (&qreg)[2][4],
                                               f32x4 (&sc)[2][2], int r, int kg) {
  bf16x8 ka[2][4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    ka[0][s] = as_bf16x8(kt[r * kKRow + 4 * s + kg]);
    ka[1][s] = as_bf16x8(kt[(16 + r) * kKRow + 4 * s + kg]);
  }
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    sc[g][0] = sc[g][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      sc[g][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[0][s], qreg[g][s], sc[g][0], 0, 0, 0);
      sc[g][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[1][s], qreg[g][s], sc[g][1], 0, 0, 0);
    }
  }
}

// O^T += V^T . P^T and l += 1 . P^T for the probabilities `pb` of one tile whose
// transposed V is `vt`.  Every element of lacc[g] of a lane is the sum over all
// 32 keys of the tile for the lane's query row: a ones-row times P^T on the
// matrix core, from the same bf16 probabilities as the numerator.
__device__ __forceinline__ void accumulate_tile(const uint4* vt, const bf16x8 (&pb)[2],
                                                f32x4 (&acc)[2][8], f32x4 (&lacc)[2], int r,
                                                int kg) {
  bf16x8 va[8];
#pragma unroll
  for (int jd = 0; jd < 8; ++jd) va[jd] = as_bf16x8(vt[(jd * 4 + kg) * kPieces + r]);
  const uint32_t one2 = 0x3F803F80u;   // two bf16 ones
  const bf16x8 ones = as_bf16x8(make_uint4(one2, one2, one2, one2));
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    lacc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[g], lacc[g], 0, 0, 0);
#pragma unroll
    for (int jd = 0; jd < 8; ++jd)
      acc[g][jd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[jd], pb[g], acc[g][jd], 0, 0, 0);
  }
}

// Probabilities of one tile from its scores (fp32 online softmax on the
// accumulator layout), already in B-operand layout.
//   m_run[g]  reference point of the exponentials, mneg[g] = -m_run * sl2.
// MASK: entries beyond `row_limit + 16*g + r` (causal) or `key_limit` (end of
// the sequence), both relative to the first key of the tile, weigh exactly 0.
// Must run after the previous tile has been accumulated: moving the reference
// point rescales acc and lacc.
template <bool MASK>
__device__ __forceinline__ void probabilities_of_tile(f32x4 (&sc)[2][2], bf16x8 (&pb)[2],
                                                      f32x4 (&acc)[2][8], f32x4 (&lacc)[2],
                                                      float (&m_run)[2], float (&mneg)[2],
                                                      float sl2, int r, int kg, int row_limit,
                                                      int key_limit) {
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    f32x4& s0 = sc[g][0];
    f32x4& s1 = sc[g][1];
    // lane = (query row r of the group, key group kg): keys 4*kg + e and
    // 16 + 4*kg + e of the tile; `limit` = last key of the tile the row may see
    const int limit = MASK ? min(row_limit + 16 * g + r, key_limit) : 0;
    if (MASK) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (4 * kg + e > limit) s0[e] = kNegBig;
        if (16 + 4 * kg + e > limit) s1[e] = kNegBig;
      }
    }
    // Lazy running max: the reference point of the exponentials only moves
    // when some lane's maximum exceeds it by more than 2^kLazyLog2 (a
    // wave-uniform decision taken on each lane's own 8 keys, so most tiles need
    // neither a cross-lane reduction nor a rescale of O^T and l).
    // Probabilities may then exceed 1 (by at most that factor); the final O / l
    // is unchanged because both carry the same reference.
    float mx = max_of8(s0, s1);
    if (__any(fmaf(mx, sl2, mneg[g]) > kLazyLog2)) {
      mx = max2(mx, __shfl_xor(mx, 16, 64));
      mx = max2(mx, __shfl_xor(mx, 32, 64));
      const float m_new = max2(m_run[g], mx);
      const float alpha = __builtin_amdgcn_exp2f((m_run[g] - m_new) * sl2);
      m_run[g] = m_new;
      mneg[g] = -m_new * sl2;
      lacc[g] *= alpha;
#pragma unroll
      for (int jd = 0; jd < 8; ++jd) acc[g][jd] *= alpha;
    }
    float p0[4], p1[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      p0[e] = __builtin_amdgcn_exp2f(fmaf(s0[e], sl2, mneg[g]));
      p1[e] = __builtin_amdgcn_exp2f(fmaf(s1[e], sl2, mneg[g]));
    }
    if (MASK) {
      // masked entries weigh exactly 0 whatever the scale and even for a row
      // whose reference point is still the initial one
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (4 * kg + e > limit) p0[e] = 0.f;
        if (16 + 4 * kg + e > limit) p1[e] = 0.f;
      }
    }
    uint4 pbits;
    pbits.x = pack_bf16x2(p0[0], p0[1]);
    pbits.y = pack_bf16x2(p0[2], p0[3]);
    pbits.z = pack_bf16x2(p1[0], p1[1]);
    pbits.w = pack_bf16x2(p1[2], p1[3]);
    pb[g] = as_bf16x8(pbits);
  }
}

struct PrefillArgs {
  const uint4* q;       // [Tq, Hq, 16] pieces
  const uint4* k;       // [Tk, Hkv, 16] pieces
  const uint4* v;
  uint4* out;           // [Tq, Hq, 16] pieces
  const int32_t* cu_q;  // [B + 1]
  const int32_t* cu_k;  // [B + 1]
  int batch, num_heads, num_kv_heads, group;
  float scale_log2e;
};

// grid.x = 8 * ceil(tile bound * Hq / 8) workgroups (see the work-item mapping below).
__global__ __launch_bounds__(kWaves * 64, 2) void prefill_attention_kernel(PrefillArgs a,
                                                                        int num_tiles_bound) {
  __shared__ uint4 k_lds[2][kKeys * kKRow];
  __shared__ uint4 vt_lds[2][8 * 4 * kPieces];   // [dim-in-piece jd][key group][piece]

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int r = lane & 15;
  const int kg = lane >> 4;
  const const_i32_ptr cu_q = (const_i32_ptr)(uintptr_t)a.cu_q;
  const const_i32_ptr cu_k = (const_i32_ptr)(uintptr_t)a.cu_k;

  // Work item -> workgroup, XCD-aware.  Consecutive workgroup ids land on
  // different XCDs (8 of them, each with its own L2), so the work list is cut
  // into 8 contiguous parts and workgroup id L takes item (L % 8) * part + L / 8:
  // one XCD then walks neighbouring items.  Items are ordered (kv head, query
  // tile, query head of the group): neighbours share the K/V rows of one
  // (sequence, kv head), which stay in that XCD's L2 instead of being fetched
  // by all eight.  Later tiles of a sequence have more keys to walk and come
  // first.
  const int total_items = num_tiles_bound * a.num_heads;
  const int part = (total_items + 7) / 8;
  const int item = ((int)blockIdx.x % 8) * part + (int)blockIdx.x / 8;
  if (item >= total_items) return;
  const int per_kv_head = num_tiles_bound * a.group;
  const int kvh = item / per_kv_head;
  const int in_kv = item - kvh * per_kv_head;
  const int tile_id = num_tiles_bound - 1 - in_kv / a.group;
  const int head = kvh * a.group + in_kv % a.group;
  int seq = -1, q0 = 0;
  {
    int before = 0;
    for (int s = 0; s < a.batch; ++s) {
      const int len = cu_q[s + 1] - cu_q[s];
      const int nt = (max(len, 0) + kBM - 1) / kBM;
      if (tile_id < before + nt) {
        seq = s;
        q0 = (tile_id - before) * kBM;
        break;
      }
      before += nt;
    }
  }
  if (seq < 0) return;   // beyond the real number of tiles
  const int q_base = cu_q[seq], len_q = cu_q[seq + 1] - q_base;
  const int k_base = cu_k[seq], len_k = max(cu_k[seq + 1] - k_base, 0);
  const int q_end = min(q0 + kBM, len_q);           // rows [q0, q_end) are real
  const int k_end = min(len_k, q_end);              // keys [0, k_end) are visible to some row
  const int nsteps = (k_end + kKeys - 1) / kKeys;

  // ---- Q^T of both column groups as B operands: column r of group g is row
  // q0 + 32*wave + 16*g + r; rows beyond the sequence are zero ----
  bf16x8 qreg[2][4];
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const int row = q0 + kRowsPerWave * wave + 16 * g + r;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    const uint4* qrow =
        a.q + ((int64_t)(q_base + min(row, len_q - 1)) * a.num_heads + head) * kPieces;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint4 t = qrow[4 * s + kg];
      qreg[g][s] = as_bf16x8(row < len_q ? t : zero);
    }
  }

  const uint32_t row_bytes = (uint32_t)a.num_kv_heads * (kD * 2);
  const char* k_head =
      reinterpret_cast<const char*>(a.k + ((int64_t)k_base * a.num_kv_heads + kvh) * kPieces);
  const char* v_head =
      reinterpret_cast<const char*>(a.v + ((int64_t)k_base * a.num_kv_heads + kvh) * kPieces);

  uint4 kld0, kld1, vld0, vld1;
  // V is loaded by lane = (piece low 3 bits, slot pair qd, piece high bit): the
  // first 32 lanes then write 8 pieces x 4 slot pairs = 32 different LDS banks
  const TileLoader ld = {k_head, v_head, row_bytes, k_end - 1, tid, wave,
                         (lane & 7) | ((lane >> 5) << 3), (lane >> 3) & 3};

  const float sl2 = a.scale_log2e;
  f32x4 acc[2][8], lacc[2];
  float m_run[2], mneg[2];
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    m_run[g] = kNegBig;
    mneg[g] = -kNegBig * sl2;
    lacc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int jd = 0; jd < 8; ++jd) acc[g][jd] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // Software pipeline over the tiles: iteration i computes the scores of tile i
  // on the matrix core, then accumulates tile i-1 (probabilities kept from the
  // previous iteration) while the vector ALU turns the scores of tile i into
  // probabilities.  So K of tile i and V^T of tile i-1 are read in iteration i:
  // the K buffers run one tile ahead of the V^T buffers.  At the top of
  // iteration i the staging registers hold K of tile i+1 and V of tile i.
  const int wave_row0 = q0 + kRowsPerWave * wave;   // first query row of this wave
  {
    // V^T "of tile -1" (probabilities are zero there, but 0 * NaN is not 0)
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    vt_lds[1][tid] = zero;
    vt_lds[1][tid + kWaves * 64] = zero;
  }
  if (nsteps > 0) {
    ld.issue_k(0, kld0, kld1);
    ld.issue_v(0, vld0, vld1);
    ld.stage_k(k_lds[0], kld0, kld1);
    if (nsteps > 1) ld.issue_k(1, kld0, kld1);
  }
  __syncthreads();

  // Tiles of this wave, in order: plain ones (every key visible to every row),
  // masked ones (the diagonal tile, or one that reaches past the last key),
  // then tiles whose keys no row of the wave sees, where it only helps to load.
  // Separate loops rather than a branch inside one keep the accumulators in place.
  const int n_active = min(nsteps, wave_row0 / kKeys + 1);
  const int n_plain = min(min(wave_row0, k_end) / kKeys, n_active);

  // Stage V^T of tile i and K of tile i+1 (their buffers were last read one
  // iteration ago, before the previous barrier) and fetch the tiles after them.
#define NVJ_STAGE_TILES(i)                                        \
  do {                                                            \
    ld.stage_v(vt_lds[(i) & 1], vld0, vld1);                      \
    if ((i) + 1 < nsteps) {                                       \
      ld.stage_k(k_lds[((i) + 1) & 1], kld0, kld1);               \
      ld.issue_v((i) + 1, vld0, vld1);                            \
      if ((i) + 2 < nsteps) ld.issue_k((i) + 2, kld0, kld1);      \
    }                                                             \
  } while (0)

  f32x4 sc[2][2];
  bf16x8 pb[2];
  pb[0] = pb[1] = as_bf16x8(make_uint4(0u, 0u, 0u, 0u));
  int i = 0;
  for (; i < n_plain; ++i) {
    scores_of_tile(k_lds[i & 1], qreg, sc, r, kg);
    NVJ_STAGE_TILES(i);
    accumulate_tile(vt_lds[(i & 1) ^ 1], pb, acc, lacc, r, kg);
    probabilities_of_tile<false>(sc, pb, acc, lacc, m_run, mneg, sl2, r, kg, 0, 0);
    __syncthreads();
  }
  for (; i < n_active; ++i) {
    const int ks = i * kKeys;
    scores_of_tile(k_lds[i & 1], qreg, sc, r, kg);
    NVJ_STAGE_TILES(i);
    accumulate_tile(vt_lds[(i & 1) ^ 1], pb, acc, lacc, r, kg);
    probabilities_of_tile<true>(sc, pb, acc, lacc, m_run, mneg, sl2, r, kg, wave_row0 - ks,
                                k_end - 1 - ks);
    __syncthreads();
  }
  // the last tile of the wave is still to be accumulated; its V^T stays in
  // place until the staging of the iteration after this one
  if (n_active > 0) accumulate_tile(vt_lds[(n_active - 1) & 1], pb, acc, lacc, r, kg);
  for (; i < nsteps; ++i) {
    NVJ_STAGE_TILES(i);
    __syncthreads();
  }
#undef NVJ_STAGE_TILES

  // ---- epilogue: acc[g][jd][e] is O[row][dim = 32*kg + 8*e + jd] ----
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const float l = lacc[g][0];   // already summed over every key of the row
    const int row = wave_row0 + 16 * g + r;
    if (row < len_q) {
      const float inv = l > 0.f ? 1.0f / l : 0.f;   // no visible key at all -> zeros
      uint4* orow = a.out + ((int64_t)(q_base + row) * a.num_heads + head) * kPieces + 4 * kg;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint4 o;
        o.x = pack_bf16x2(acc[g][0][e] * inv, acc[g][1][e] * inv);
        o.y = pack_bf16x2(acc[g][2][e] * inv, acc[g][3][e] * inv);
        o.z = pack_bf16x2(acc[g][4][e] * inv, acc[g][5][e] * inv);
        o.w = pack_bf16x2(acc[g][6][e] * inv, acc[g][7][e] * inv);
        orow[e] = o;
      }
    }
  }
}

}  // namespace

extern "C" int nvj_prefill_attention_launch(void* stream, const void* q, const void* k,
                                            const void* v, const int32_t* cu_seqlens_q,
                                            const int32_t* cu_seqlens_k, void* out,
                                            int32_t total_q_tokens, int32_t batch,
                                            int32_t num_heads, int32_t num_kv_heads,
                                            int32_t head_dim, float scale) {
  if (total_q_tokens < 0 || batch < 0 || num_heads <= 0 || num_kv_heads <= 0)
    return NVJ_ERR_BAD_SHAPE;
  if (num_heads % num_kv_heads != 0) return NVJ_ERR_BAD_SHAPE;
  if (head_dim != kD) return NVJ_ERR_UNSUPPORTED;
  if (num_kv_heads > 32768) return NVJ_ERR_UNSUPPORTED;   // a key row stays below 2^24 bytes
  if (!(scale >= 0.f)) return NVJ_ERR_BAD_SHAPE;   // the running max assumes a non-negative scale
  if (total_q_tokens == 0 || batch == 0) return NVJ_OK;
  if (!q || !k || !v || !cu_seqlens_q || !cu_seqlens_k || !out) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) |
       reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(out)) & 15u)
    return NVJ_ERR_BAD_SHAPE;
  PrefillArgs a;
  a.q = static_cast<const uint4*>(q);
  a.k = static_cast<const uint4*>(k);
  a.v = static_cast<const uint4*>(v);
  a.out = static_cast<uint4*>(out);
  a.cu_q = cu_seqlens_q;
  a.cu_k = cu_seqlens_k;
  a.batch = batch;
  a.num_heads = num_heads;
  a.num_kv_heads = num_kv_heads;
  a.group = num_heads / num_kv_heads;
  a.scale_log2e = scale * kLog2e;
  // every sequence adds at most one partly filled tile
  const int64_t tiles = (int64_t)total_q_tokens / kBM + batch;
  if (tiles > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  const int64_t items = tiles * num_heads;
  if (items > INT32_MAX - 8) return NVJ_ERR_BAD_SHAPE;
  const unsigned grid = (unsigned)((items + 7) / 8 * 8);
  prefill_attention_kernel<<<dim3(grid), dim3(kWaves * 64), 0,
                             static_cast<hipStream_t>(stream)>>>(a, (int)tiles);
  return hipGetLastError() == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

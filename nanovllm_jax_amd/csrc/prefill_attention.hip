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
// 32 at a time.  The K rows and the V rows of a tile go from global memory
// straight into LDS (global_load_lds_dwordx4: no staging registers, no LDS
// write instructions), row-major with the 16-byte pieces of a row permuted so
// that the reads below are free of bank conflicts, in rings of 4 tiles each,
// fetched two tiles ahead; one barrier per tile:
//   * K is read back with ds_read_b128 as the A operand of
//     S^T[key, q] = K . Q^T  (v_mfma_f32_16x16x32_bf16, Q^T of both groups in
//     registers for the whole tile);
//   * V is read back with the transposing LDS read (ds_read_b64_tr_b16), which
//     hands each lane four keys of one head dimension: the A operand of
//     O^T[dim, q] += V^T . P^T.
// Softmax is the fp32 online form on the accumulator layout; P^T comes out of
// the S^T accumulators already in B-operand layout (same reduction-slot <-> key
// map as the decode kernel).  Only tiles that touch the diagonal are masked.
// The loop is software-pipelined: the scores of tile i are issued to the matrix
// core, then tile i-1 is accumulated while the vector ALU turns the scores of
// tile i into probabilities.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch.h"
#include "nvj_paged_attn.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kD = 128;
constexpr int kPieces = 16;          // 16-byte pieces per (position, head) row
// 2 groups x 4 waves (128 query rows, two workgroups per CU) measured fastest:
// 4 groups x 4 waves (one wave per SIMD, accumulators in AGPRs) and 8-wave
// workgroups (1 or 2 groups) were 5-20 % slower.
constexpr int kGroups = 2;           // column groups of 16 query rows per wave
constexpr int kWaves = 4;
constexpr int kRowsPerWave = 16 * kGroups;
constexpr int kBM = kRowsPerWave * kWaves;   // query rows per workgroup
constexpr int kKeys = 32;            // keys per step
constexpr int kTileBytes = kKeys * kD * 2;   // one K or V tile in LDS: 32 rows of 256 bytes
// Both rings hold 4 tiles, tile t in slot t % 4: iteration i reads K of tile i and
// V of tile i-1 while tiles i+1 (landing) and i+2 (just issued) are on their way.
// A ring of 3 would do for K; 4 makes the slot of every tile of an iteration a
// function of i % 4, so that a loop unrolled 4 times has every LDS offset as an
// instruction immediate.
constexpr int kKStages = 4;
constexpr int kVStages = 4;
constexpr float kNegBig = -1.0e30f;
constexpr float kLazyLog2 = 8.0f;    // running max moves only for gains above 2^8
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// The element type of q, k, v and out: bf16 (F16 = false) or IEEE half.  The
// kernel moves 16-bit patterns (held as bf16x8 whatever they mean); only the
// matrix instruction, the rounding of probabilities and output and the
// constant 1 depend on the type.
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
template <bool F16> struct Elem;
template <> struct Elem<false> {
  static constexpr uint32_t kOnes = 0x3F803F80u;   // two bf16 ones
  static __device__ __forceinline__ f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    bf16x2 p = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, p);
  }
};
template <> struct Elem<true> {
  static constexpr uint32_t kOnes = 0x3C003C00u;   // two half ones
  static __device__ __forceinline__ f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
    f16x2 p = {(_Float16)lo, (_Float16)hi};   // round to nearest even
    return __builtin_bit_cast(uint32_t, p);
  }
};

typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;

// reduction slot j of key group kg stands for this key of the 32-key step
__device__ __forceinline__ int slot_key(int kg, int j) {
  return j < 4 ? 4 * kg + j : 16 + 4 * kg + (j - 4);
}

typedef __attribute__((address_space(3))) char* lds_ptr;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

// LDS layout of a tile: row R (key R of the tile) at byte 256 * R, its 16-byte
// piece p at position p ^ (R & 15) for K and p ^ (2 * (R & 7)) for V.
//   K read (ds_read_b128): the 16 lanes of a key group read one piece of 16
//     different rows -> 16 different positions.
//   V read (ds_read_b64_tr_b16): the 16 lanes of a key group read four 8-byte
//     chunks of each of 4 rows -> 16 different 8-byte slots modulo 128 bytes.
__device__ __forceinline__ int k_position(int row, int piece) { return piece ^ (row & 15); }
__device__ __forceinline__ int v_position(int row, int piece) { return piece ^ (2 * (row & 7)); }

// One 16-byte global -> LDS copy per lane: lane l's piece lands at
// lds_base + 16 * l (lds_base wave-uniform), fetched from base + offset.
// Counts in vmcnt like any load; the compiler does not see it as one, so the
// waits are written out by hand (wait_tiles_in_flight).
__device__ __forceinline__ void copy16_to_lds(const char* base, uint32_t offset,
                                              uint32_t lds_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(lds_base), "v"(offset), "s"(base)
      : "memory");
}

// Cooperative tile copies of a workgroup.  A tile is 512 pieces of K and 512 of
// V; each wave copies its share of the rows of both (8 rows with 4 waves), 4
// rows = 1024 contiguous LDS bytes per instruction.  Lane l of instruction j of
// wave w writes position l % 16 of row 8w + 4j + l / 16 and fetches the piece
// that belongs there.  Rows are clamped to the last visible key, so nothing at or beyond
// k_end is read.
constexpr int kCopyRowsPerWave = kKeys / kWaves;   // rows of a tile one wave copies
static_assert(kCopyRowsPerWave % 4 == 0, "one copy instruction covers 4 rows");
// Packed rows: key s of the sequence is row s behind k_head / v_head.  Paged
// (PAGED): k_head / v_head point at this kv head inside row 0 of the caches and
// key s is row table[s / block_size] * block_size + s % block_size; a tile of 32
// keys never leaves its page (block_size is a multiple of 32), so one scalar
// table lookup per tile gives the base and the lanes keep their row offsets.
template <bool PAGED>
struct TileCopier {
  const char* k_head;   // first key row of the sequence for this kv head
  const char* v_head;
  uint32_t row_bytes;   // bytes between consecutive keys; < 2^24 (checked by the host)
  uint32_t k_lds, v_lds;   // LDS byte addresses of the two rings
  int last_key, last_tile, wave, lane;
  const_i32_ptr table;  // PAGED: this sequence's row of the block tables
  int block_size, num_blocks;

  __device__ __forceinline__ void issue(int tile, int k_stage, int v_stage) const {
    tile = min(tile, last_tile);   // past the end: fetch the last tile again (same instruction count)
    const int ks = tile * kKeys;
    const int cap = last_key - ks;   // >= 0: a tile starts at a visible key
    size_t first_row = (size_t)ks;
    if (PAGED) {
      const int page = ks / block_size;
      const int phys = min(max(table[page], 0), num_blocks - 1);
      first_row = (size_t)phys * block_size + (ks - page * block_size);
    }
    const char* kb = k_head + first_row * row_bytes;
    const char* vb = v_head + first_row * row_bytes;
#pragma unroll
    for (int j = 0; j < kCopyRowsPerWave / 4; ++j) {
      const int row = kCopyRowsPerWave * wave + 4 * j + (lane >> 4);
      const uint32_t row_off = __umul24(min(row, cap), row_bytes);
      const uint32_t dst = (uint32_t)(kCopyRowsPerWave / 4 * wave + j) * 1024u;
      copy16_to_lds(kb, row_off + 16u * k_position(row, lane & 15),
                    k_lds + (uint32_t)k_stage * kTileBytes + dst);
      copy16_to_lds(vb, row_off + 16u * v_position(row, lane & 15),
                    v_lds + (uint32_t)v_stage * kTileBytes + dst);
    }
  }

  // The same for a tile all of whose 32 keys exist (tile < last_tile): the
  // lanes' offsets do not depend on the tile and are computed once (lane_offsets).
  __device__ __forceinline__ void lane_offsets(uint32_t (&koff)[kCopyRowsPerWave / 4],
                                               uint32_t (&voff)[kCopyRowsPerWave / 4]) const {
#pragma unroll
    for (int j = 0; j < kCopyRowsPerWave / 4; ++j) {
      const int row = kCopyRowsPerWave * wave + 4 * j + (lane >> 4);
      const uint32_t row_off = __umul24(row, row_bytes);
      koff[j] = row_off + 16u * k_position(row, lane & 15);
      voff[j] = row_off + 16u * v_position(row, lane & 15);
    }
  }
  template <int STAGE>
  __device__ __forceinline__ void issue_full(int tile, const uint32_t (&koff)[kCopyRowsPerWave / 4],
                                             const uint32_t (&voff)[kCopyRowsPerWave / 4]) const {
    const int ks = tile * kKeys;
    size_t first_row = (size_t)ks;
    if (PAGED) {
      const int page = ks / block_size;
      const int phys = min(max(table[page], 0), num_blocks - 1);
      first_row = (size_t)phys * block_size + (ks - page * block_size);
    }
    const char* kb = k_head + first_row * row_bytes;
    const char* vb = v_head + first_row * row_bytes;
#pragma unroll
    for (int j = 0; j < kCopyRowsPerWave / 4; ++j) {
      const uint32_t dst = (uint32_t)(kCopyRowsPerWave / 4 * wave + j) * 1024u;
      copy16_to_lds(kb, koff[j], k_lds + (uint32_t)STAGE * kTileBytes + dst);
      copy16_to_lds(vb, voff[j], v_lds + (uint32_t)STAGE * kTileBytes + dst);
    }
  }
};
constexpr int kCopiesPerTile = 2 * (kCopyRowsPerWave / 4);   // copy16_to_lds calls of one lane per tile

// Blocks until at most `tiles` of this lane's most recent tile copies are still
// in flight (vmcnt counts the copies in order).
template <int TILES>
__device__ __forceinline__ void wait_tiles_in_flight() {
  static_assert(TILES == 0 || TILES == 1, "vmcnt immediates below");
  static_assert(kCopiesPerTile == 4 || kCopiesPerTile == 2, "vmcnt immediates below");
  if (TILES == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else if (kCopiesPerTile == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
}

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
// kaddr[s] is the lane's LDS address of its piece 4*s + kg of row r of ring slot
// 0 (k_read_addresses); `slot_bytes` selects the ring slot.
template <bool F16>
__device__ __forceinline__ void scores_of_tile(const lds_ptr (&kaddr)[4], int slot_bytes,
                                               const bf16x8 (&qreg)[kGroups][4],
                                               f32x4 (&sc)[kGroups][2]) {
  bf16x8 ka[2][4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    // rows r and 16 + r share a position: (16 + r) & 15 == r
    ka[0][s] = *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>(
        kaddr[s] + slot_bytes);
    ka[1][s] = *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>(
        kaddr[s] + slot_bytes + 16 * 256);
  }
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    sc[g][0] = sc[g][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      sc[g][0] = Elem<F16>::mfma(ka[0][s], qreg[g][s], sc[g][0]);
      sc[g][1] = Elem<F16>::mfma(ka[1][s], qreg[g][s], sc[g][1]);
    }
  }
}
__device__ __forceinline__ void k_read_addresses(lds_ptr k_lds, int r, int kg, lds_ptr (&kaddr)[4]) {
#pragma unroll
  for (int s = 0; s < 4; ++s) kaddr[s] = k_lds + 256 * r + 16 * k_position(r, 4 * s + kg);
}

// O^T += V^T . P^T and l += 1 . P^T for the probabilities `pb` of one tile whose
// V rows are at `vt`.  Operand jd covers head dimensions 16*jd .. 16*jd + 15.
// ds_read_b64_tr_b16 works on groups of 16 lanes: source lane s = 4a + b of a
// group points at 4 consecutive bf16 (b selects which 4 of the 16 dimensions)
// of row a; result lane 4b + j receives, as element a, the j-th of those from
// source lane 4a + b.  With row a = key 4*kg + a of the tile (then 16 + 4*kg + a
// for the second read) lane i of the group ends up with keys of reduction
// slots 0..3 (then 4..7) of dimension 16*jd + i: the A operand.
// Every element of lacc[g] of a lane is the sum over all 32 keys of the tile for
// the lane's query row: a ones-row times P^T on the matrix core, from the same
// bf16 probabilities as the numerator.
// vaddr[jd] is the lane's LDS address for operand jd in ring slot 0
// (v_read_addresses); `slot_bytes` selects the ring slot.
template <bool F16>
__device__ __forceinline__ void accumulate_tile(const lds_ptr (&vaddr)[8], int slot_bytes,
                                                const bf16x8 (&pb)[kGroups],
                                                f32x4 (&acc)[kGroups][8], f32x4 (&lacc)[kGroups]) {
  bf16x8 va[8];
#pragma unroll
  for (int jd = 0; jd < 8; ++jd) {
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        reinterpret_cast<__attribute__((address_space(3))) bf16x4*>(vaddr[jd] + slot_bytes));
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        reinterpret_cast<__attribute__((address_space(3))) bf16x4*>(vaddr[jd] + slot_bytes +
                                                                      16 * 256));
    va[jd] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
  const uint32_t one2 = Elem<F16>::kOnes;
  const bf16x8 ones = as_bf16x8(make_uint4(one2, one2, one2, one2));
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    lacc[g] = Elem<F16>::mfma(ones, pb[g], lacc[g]);
#pragma unroll
    for (int jd = 0; jd < 8; ++jd)
      acc[g][jd] = Elem<F16>::mfma(va[jd], pb[g], acc[g][jd]);
  }
}
__device__ __forceinline__ void v_read_addresses(lds_ptr v_lds, int r, int kg, lds_ptr (&vaddr)[8]) {
  const int row = 4 * kg + (r >> 2);   // (16 + row) & 7 == row & 7: both reads share positions
  const int chunk = r & 3;             // 8-byte chunk of the 32 bytes of a dimension group
#pragma unroll
  for (int jd = 0; jd < 8; ++jd)
    vaddr[jd] = v_lds + 256 * row + 16 * v_position(row, 2 * jd + (chunk >> 1)) + 8 * (chunk & 1);
}

// Probabilities of one tile from its scores (fp32 online softmax on the
// accumulator layout), already in B-operand layout.
//   m_run[g]  reference point of the exponentials, mneg[g] = -m_run * sl2.
// MASK: entries beyond `row_limit + 16*g + r` (causal) or `key_limit` (end of
// the sequence), both relative to the first key of the tile, weigh exactly 0.
// Must run after the previous tile has been accumulated: moving the reference
// point rescales acc and lacc.
template <bool MASK, bool F16>
__device__ __forceinline__ void probabilities_of_tile(f32x4 (&sc)[kGroups][2], bf16x8 (&pb)[kGroups],
                                                      f32x4 (&acc)[kGroups][8], f32x4 (&lacc)[kGroups],
                                                      float (&m_run)[kGroups], float (&mneg)[kGroups],
                                                      float sl2, int r, int kg, int row_limit,
                                                      int key_limit) {
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
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
    pbits.x = Elem<F16>::pack2(p0[0], p0[1]);
    pbits.y = Elem<F16>::pack2(p0[2], p0[3]);
    pbits.z = Elem<F16>::pack2(p1[0], p1[1]);
    pbits.w = Elem<F16>::pack2(p1[2], p1[3]);
    pb[g] = as_bf16x8(pbits);
  }
}

struct PrefillArgs {
  const uint4* q;       // [Tq, Hq, 16] pieces
  const uint4* k;       // [Tk, Hkv, 16] pieces
  const uint4* v;
  uint4* out;           // [Tq, Hq, 16] pieces
  const int32_t* cu_q;  // [B + 1]
  const int32_t* cu_k;  // [B + 1]; paged: the keys of a sequence, cached and new together
  int batch, num_heads, num_kv_heads, group;
  float scale_log2e;
  // paged only: k and v are the caches [num_blocks, block_size, Hkv, 16] pieces
  const int32_t* block_tables;   // [B, max_blocks]
  int block_size, max_blocks, num_blocks;
};

// grid.x = 8 * ceil(tile bound * Hq / 8) workgroups (see the work-item mapping below).
// PAGED: keys and values come from the block-paged cache through block_tables,
// sequence i has len_k = cu_k[i+1] - cu_k[i] keys, and its len_q query rows are the
// LAST len_q positions of the sequence (row j sees keys <= len_k - len_q + j):
// prompt rows behind a cached prefix.  Otherwise: packed rows, both counted
// from the start of the sequence as the reference's mask does.
template <bool F16, bool PAGED>
__global__ __launch_bounds__(kWaves * 64, kGroups <= 2 ? 2 : 1) void prefill_attention_kernel(PrefillArgs a,
                                                                        int num_tiles_bound) {
  __shared__ uint4 k_ring[kKStages * kTileBytes / 16];
  __shared__ uint4 v_ring[kVStages * kTileBytes / 16];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int r = lane & 15;
  const int kg = lane >> 4;
  const const_i32_ptr cu_q = (const_i32_ptr)(uintptr_t)a.cu_q;

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
  const int head = kvh * a.group + in_kv % a.group;
  // Query tiles are numbered sequence by sequence.  A wave looks at 64 sequences
  // at a time, one per lane, with the offsets of 256 sequences fetched together
  // (one round trip per 256 sequences; a loop over the sequences one by one cost
  // a batch of 128 short prompts more than its tiles).  First the real number of
  // tiles: the work list was sized for a bound, and the items beyond the real
  // tiles sit at its end, where they delay nothing.  The real tiles are walked
  // from the last one down (the later tiles of a sequence have more keys).
  int nt4[4], qb4[4], ql4[4], kb4[4], kl4[4];
  auto load_offsets = [&](int base) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int s = min(base + 64 * k + lane, a.batch - 1);
      qb4[k] = a.cu_q[s];
      ql4[k] = a.cu_q[s + 1] - qb4[k];
      kb4[k] = a.cu_k[s];
      kl4[k] = a.cu_k[s + 1] - kb4[k];
      nt4[k] = base + 64 * k + lane < a.batch ? (max(ql4[k], 0) + kBM - 1) / kBM : 0;
    }
  };
  int real_tiles = 0;
  for (int base = 0; base < a.batch; base += 256) {
    load_offsets(base);
    int sum = nt4[0] + nt4[1] + nt4[2] + nt4[3];
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) sum += __shfl_xor(sum, d, 64);
    real_tiles += sum;
  }
  real_tiles = __builtin_amdgcn_readfirstlane(real_tiles);
  if (in_kv / a.group >= real_tiles) return;   // beyond the real number of tiles
  const int tile_id = real_tiles - 1 - in_kv / a.group;
  int seq = -1, q0 = 0;
  int q_base = 0, len_q = 0, k_first = 0, k_count = 0;   // of that sequence, from the same loads
  {
    int before = 0;   // tiles of the sequences in front of this group of 64
    for (int base = 0; base < a.batch && seq < 0; base += 256) {
      if (a.batch > 256) load_offsets(base);   // (a smaller batch is still in registers)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (base + 64 * k < a.batch && seq < 0) {
          const int nt = nt4[k];
          int incl = nt;   // tiles up to and including this lane's sequence
#pragma unroll
          for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d, 64);
            if (lane >= d) incl += up;
          }
          const unsigned long long hit =
              __ballot(nt > 0 && tile_id >= before + incl - nt && tile_id < before + incl);
          if (hit != 0ull) {
            const int src = __builtin_ctzll(hit);
            seq = base + 64 * k + src;
            q0 = (tile_id - before - __shfl(incl - nt, src, 64)) * kBM;
            q_base = __shfl(qb4[k], src, 64);
            len_q = __shfl(ql4[k], src, 64);
            k_first = __shfl(kb4[k], src, 64);
            k_count = __shfl(kl4[k], src, 64);
          }
          before += __shfl(incl, 63, 64);
        }
      }
    }
    seq = __builtin_amdgcn_readfirstlane(seq);
    q0 = __builtin_amdgcn_readfirstlane(q0);
    q_base = __builtin_amdgcn_readfirstlane(q_base);
    len_q = __builtin_amdgcn_readfirstlane(len_q);
    k_first = __builtin_amdgcn_readfirstlane(k_first);
    k_count = __builtin_amdgcn_readfirstlane(k_count);
  }
  if (seq < 0) return;   // (cannot happen: tile_id is a real tile)
  const int k_base = PAGED ? 0 : k_first;
  const int len_k = PAGED ? min(max(k_count, 0), a.max_blocks * a.block_size) : max(k_count, 0);
  // key position of query row 0: rows are the tail of the sequence when paged
  const int off = PAGED ? max(len_k - len_q, 0) : 0;
  const int q_end = min(q0 + kBM, len_q);           // rows [q0, q_end) are real
  const int k_end = min(len_k, off + q_end);        // keys [0, k_end) are visible to some row
  const int nsteps = (k_end + kKeys - 1) / kKeys;

  // ---- Q^T of both column groups as B operands: column r of group g is row
  // q0 + 32*wave + 16*g + r; rows beyond the sequence are zero ----
  bf16x8 qreg[kGroups][4];
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
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
  const const_i32_ptr table =
      PAGED ? (const_i32_ptr)(uintptr_t)(a.block_tables + (int64_t)seq * a.max_blocks) : cu_q;

  const lds_ptr k_lds = (lds_ptr)k_ring;
  const lds_ptr v_lds = (lds_ptr)v_ring;
  const TileCopier<PAGED> copier = {k_head, v_head, row_bytes, (uint32_t)(uintptr_t)k_lds,
                                    (uint32_t)(uintptr_t)v_lds, k_end - 1, nsteps - 1, wave, lane,
                                    table, a.block_size, a.num_blocks};

  const float sl2 = a.scale_log2e;
  f32x4 acc[kGroups][8], lacc[kGroups];
  float m_run[kGroups], mneg[kGroups];
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    m_run[g] = kNegBig;
    mneg[g] = -kNegBig * sl2;
    lacc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int jd = 0; jd < 8; ++jd) acc[g][jd] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // Software pipeline over the tiles: iteration i issues the scores of tile i to
  // the matrix core, then accumulates tile i-1 (probabilities kept from the
  // previous iteration) while the vector ALU turns the scores of tile i into
  // probabilities.  Iteration i therefore reads K of tile i and V of tile i-1,
  // and starts the copies of tile i+2 into the ring slots last read in iteration
  // i-1 (K of tile i-1, V of tile i-2).  Before the barrier that ends it, every
  // lane waits for its copies of tile i+1.
  const int wave_row0 = q0 + kRowsPerWave * wave;   // first query row of this wave
  if (nsteps > 0) {
    // V "of tile -1" (probabilities are zero there, but 0 * NaN is not 0)
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    uint4* v_before = v_ring + (kVStages - 1) * (kTileBytes / 16);
    for (int p = tid; p < kTileBytes / 16; p += kWaves * 64) v_before[p] = zero;
    copier.issue(0, 0, 0);
    copier.issue(1, 1, 1);
    wait_tiles_in_flight<1>();
  }
  __syncthreads();

  // Tiles of this wave, in order: plain ones (every key visible to every row),
  // masked ones (the diagonal tile, or one that reaches past the last key),
  // then tiles whose keys no row of the wave sees, where it only helps to copy.
  // Separate loops rather than a branch inside one keep the accumulators in place.
  const int n_active = min(nsteps, (off + wave_row0 + kRowsPerWave - 1) / kKeys + 1);
  const int n_plain = min(min(off + wave_row0, k_end) / kKeys, n_active);

  // Tile t lives in ring slot t % 4 (K and V alike).  Iteration i: scores of tile
  // i, accumulation of tile i-1, probabilities of tile i, copies of tile i+2 into
  // the slot last read in iteration i-1, wait for this lane's copies of tile i+1,
  // barrier.
  lds_ptr kaddr[4], vaddr[8];
  k_read_addresses(k_lds, r, kg, kaddr);
  v_read_addresses(v_lds, r, kg, vaddr);
  uint32_t koff[kCopyRowsPerWave / 4], voff[kCopyRowsPerWave / 4];
  copier.lane_offsets(koff, voff);

  f32x4 sc[kGroups][2];
  bf16x8 pb[kGroups];
#pragma unroll
  for (int g = 0; g < kGroups; ++g) pb[g] = as_bf16x8(make_uint4(0u, 0u, 0u, 0u));
  // Waves that issue matrix instructions go first: a wave lowers its priority
  // only while it turns scores into probabilities (vector ALU work that the
  // other wave of the SIMD can overlap with its own matrix instructions).
  __builtin_amdgcn_s_setprio(1);
#define NVJ_END_OF_TILE()       \
  do {                          \
    wait_tiles_in_flight<1>();  \
    __syncthreads();            \
  } while (0)
  // a plain tile whose ring slots are known when the code is written: every LDS
  // offset is an immediate, the copies use the lanes' precomputed offsets
#define NVJ_PLAIN_TILE_AT(S, i)                                                              \
  do {                                                                                       \
    scores_of_tile<F16>(kaddr, (S) * kTileBytes, qreg, sc);                                  \
    accumulate_tile<F16>(vaddr, (((S) + 3) & 3) * kTileBytes, pb, acc, lacc);                \
    __builtin_amdgcn_s_setprio(0);                                                           \
    probabilities_of_tile<false, F16>(sc, pb, acc, lacc, m_run, mneg, sl2, r, kg, 0, 0);     \
    __builtin_amdgcn_s_setprio(1);                                                           \
    copier.template issue_full<((S) + 2) & 3>((i) + 2, koff, voff);                          \
    NVJ_END_OF_TILE();                                                                       \
  } while (0)
  // any tile, ring slots computed at run time
#define NVJ_TILE(MASKED, i, row_limit, key_limit)                                            \
  do {                                                                                       \
    scores_of_tile<F16>(kaddr, ((i) & 3) * kTileBytes, qreg, sc);                            \
    accumulate_tile<F16>(vaddr, (((i) + 3) & 3) * kTileBytes, pb, acc, lacc);                \
    __builtin_amdgcn_s_setprio(0);                                                           \
    probabilities_of_tile<MASKED, F16>(sc, pb, acc, lacc, m_run, mneg, sl2, r, kg, row_limit, \
                                       key_limit);                                           \
    __builtin_amdgcn_s_setprio(1);                                                           \
    copier.issue((i) + 2, ((i) + 2) & 3, ((i) + 2) & 3);                                     \
    NVJ_END_OF_TILE();                                                                       \
  } while (0)

  int i = 0;
  // four plain tiles at a time while the tiles they fetch (up to i + 5) are full ones
  for (; i + 4 <= n_plain && i + 5 < nsteps - 1; i += 4) {
    NVJ_PLAIN_TILE_AT(0, i);
    NVJ_PLAIN_TILE_AT(1, i + 1);
    NVJ_PLAIN_TILE_AT(2, i + 2);
    NVJ_PLAIN_TILE_AT(3, i + 3);
  }
  for (; i < n_plain; ++i) NVJ_TILE(false, i, 0, 0);
  for (; i < n_active; ++i) {
    const int ks = i * kKeys;
    NVJ_TILE(true, i, off + wave_row0 - ks, k_end - 1 - ks);
  }
  // the last tile of the wave is still to be accumulated; its V stays in place
  // until the copies of two iterations from now
  if (n_active > 0) accumulate_tile<F16>(vaddr, ((i + 3) & 3) * kTileBytes, pb, acc, lacc);
  for (; i < nsteps; ++i) {
    copier.issue(i + 2, (i + 2) & 3, (i + 2) & 3);
    NVJ_END_OF_TILE();
  }
  wait_tiles_in_flight<0>();   // copies past the last tile are still landing in LDS
#undef NVJ_TILE
#undef NVJ_PLAIN_TILE_AT
#undef NVJ_END_OF_TILE

  // ---- epilogue: acc[g][jd][e] is O[row][dim = 16*jd + 4*kg + e] ----
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    const float l = lacc[g][0];   // already summed over every key of the row
    const int row = wave_row0 + 16 * g + r;
    if (row < len_q) {
      const float inv = l > 0.f ? 1.0f / l : 0.f;   // no visible key at all -> zeros
      uint2* orow = reinterpret_cast<uint2*>(
          a.out + ((int64_t)(q_base + row) * a.num_heads + head) * kPieces);
#pragma unroll
      for (int jd = 0; jd < 8; ++jd) {
        uint2 o;
        o.x = Elem<F16>::pack2(acc[g][jd][0] * inv, acc[g][jd][1] * inv);
        o.y = Elem<F16>::pack2(acc[g][jd][2] * inv, acc[g][jd][3] * inv);
        orow[4 * jd + kg] = o;
      }
    }
  }
}

int launch_prefill(hipStream_t stream, PrefillArgs a, bool paged, int32_t total_q_tokens,
                   int32_t dtype) {
  // every sequence adds at most one partly filled tile
  const int64_t tiles = (int64_t)total_q_tokens / kBM + a.batch;
  if (tiles > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  const int64_t items = tiles * a.num_heads;
  if (items > INT32_MAX - 8) return NVJ_ERR_BAD_SHAPE;
  const dim3 grid((unsigned)((items + 7) / 8 * 8)), block(kWaves * 64);
  const int nt = (int)tiles;
  const bool f16 = dtype == NVJ_DTYPE_F16;
  hipError_t rc;
  if (paged && f16) rc = nvj::launch(prefill_attention_kernel<true, true>, grid, block, stream, a, nt);
  else if (paged) rc = nvj::launch(prefill_attention_kernel<false, true>, grid, block, stream, a, nt);
  else if (f16) rc = nvj::launch(prefill_attention_kernel<true, false>, grid, block, stream, a, nt);
  else rc = nvj::launch(prefill_attention_kernel<false, false>, grid, block, stream, a, nt);
  return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

}  // namespace

extern "C" int nvj_prefill_attention_launch(void* stream, const void* q, const void* k,
                                            const void* v, const int32_t* cu_seqlens_q,
                                            const int32_t* cu_seqlens_k, void* out,
                                            int32_t total_q_tokens, int32_t batch,
                                            int32_t num_heads, int32_t num_kv_heads,
                                            int32_t head_dim, float scale, int32_t dtype) {
  if (dtype != NVJ_DTYPE_BF16 && dtype != NVJ_DTYPE_F16) return NVJ_ERR_BAD_DTYPE;
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
    return NVJ_ERR_ALIGNMENT;
  PrefillArgs a = {};
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
  return launch_prefill(static_cast<hipStream_t>(stream), a, false, total_q_tokens, dtype);
}

extern "C" int nvj_paged_prefill_attention_launch(
    void* stream, const void* q, const void* k_cache, const void* v_cache,
    const int32_t* block_tables, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
    void* out, int32_t total_q_tokens, int32_t batch, int32_t num_heads, int32_t num_kv_heads,
    int32_t head_dim, int32_t block_size, int32_t max_blocks, int32_t num_blocks, float scale,
    int32_t dtype) {
  if (dtype != NVJ_DTYPE_BF16 && dtype != NVJ_DTYPE_F16) return NVJ_ERR_BAD_DTYPE;
  if (total_q_tokens < 0 || batch < 0 || num_heads <= 0 || num_kv_heads <= 0 || block_size <= 0 ||
      max_blocks < 0 || num_blocks <= 0)
    return NVJ_ERR_BAD_SHAPE;
  if (num_heads % num_kv_heads != 0) return NVJ_ERR_BAD_SHAPE;
  if (head_dim != kD || block_size % kKeys != 0) return NVJ_ERR_UNSUPPORTED;
  if (num_kv_heads > 32768) return NVJ_ERR_UNSUPPORTED;   // a key row stays below 2^24 bytes
  if ((int64_t)max_blocks * block_size > INT32_MAX) return NVJ_ERR_BAD_SHAPE;
  if (!(scale >= 0.f)) return NVJ_ERR_BAD_SHAPE;
  if (total_q_tokens == 0 || batch == 0) return NVJ_OK;
  if (!q || !k_cache || !v_cache || !cu_seqlens_q || !cu_seqlens_k || !out)
    return NVJ_ERR_NULL_POINTER;
  if (max_blocks > 0 && !block_tables) return NVJ_ERR_NULL_POINTER;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_cache) |
       reinterpret_cast<uintptr_t>(v_cache) | reinterpret_cast<uintptr_t>(out)) & 15u)
    return NVJ_ERR_ALIGNMENT;
  PrefillArgs a = {};
  a.q = static_cast<const uint4*>(q);
  a.k = static_cast<const uint4*>(k_cache);
  a.v = static_cast<const uint4*>(v_cache);
  a.out = static_cast<uint4*>(out);
  a.cu_q = cu_seqlens_q;
  a.cu_k = cu_seqlens_k;
  a.batch = batch;
  a.num_heads = num_heads;
  a.num_kv_heads = num_kv_heads;
  a.group = num_heads / num_kv_heads;
  a.scale_log2e = scale * kLog2e;
  a.block_tables = block_tables;
  a.block_size = block_size;
  a.max_blocks = max_blocks;
  a.num_blocks = num_blocks;
  return launch_prefill(static_cast<hipStream_t>(stream), a, true, total_q_tokens, dtype);
}

// Device-resident decode metadata for gfx950: advance the per-sequence arrays
// of one decode step to the next step without going through the host.
//
// Stands in for ModelRunner._prepare_decode (engine/model_runner.py:334-376 of
// the reference), which rebuilds five NumPy arrays per step in a Python loop
// and copies them to the device:
//   input_ids[i]    = seq.last_token
//   positions[i]    = len(seq) - 1
//   context_lens[i] = len(seq)
//   slot_mapping[i] = seq.block_table[-1] * block_size + seq.last_block_num_tokens - 1
// Here the arrays stay in HBM; after a step has produced one token per
// sequence, every sequence grows by that token and the same formulas are
// applied in place.  Tiny integer work, one lane per sequence.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch.h"
#include "nvj_paged_attn.h"

namespace {

template <typename TokenT>
__global__ __launch_bounds__(256) void advance_decode_kernel(
    const TokenT* __restrict__ next_tokens, int32_t* __restrict__ input_ids,
    int32_t* __restrict__ positions, int32_t* __restrict__ context_lens,
    int32_t* __restrict__ slot_mapping, const int32_t* __restrict__ block_tables, int batch,
    int max_blocks, int block_size) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= batch) return;
  const int len_old = context_lens[i];
  if (len_old <= 0) {  // inactive row: stays inactive, stores nothing
    slot_mapping[i] = -1;
    return;
  }
  const int64_t len = (int64_t)len_old + 1;   // the sequence with its new token
  const int64_t last = len - 1;               // position of the token to decode
  const int64_t page_idx = last / block_size;
  int32_t slot = -1;
  if (page_idx < max_blocks) {
    const int32_t page = block_tables[(int64_t)i * max_blocks + page_idx];
    // block_table[-1] * block_size + last_block_num_tokens - 1; a page that has
    // not been assigned yet (-1 padding) or a slot beyond int32 stores nothing
    const int64_t s = (int64_t)page * block_size + last % block_size;
    if (page >= 0 && s <= INT32_MAX) slot = (int32_t)s;
  }
  if (slot < 0 || len > INT32_MAX) {   // cannot grow: keep the row as it is, store nothing
    slot_mapping[i] = -1;
    return;
  }
  input_ids[i] = (int32_t)next_tokens[i];
  positions[i] = (int32_t)last;
  context_lens[i] = (int32_t)len;
  slot_mapping[i] = slot;
}

}  // namespace

extern "C" int nvj_advance_decode_launch(void* stream, const void* next_tokens,
                                         int32_t token_bytes, int32_t* input_ids,
                                         int32_t* positions, int32_t* context_lens,
                                         int32_t* slot_mapping, const int32_t* block_tables,
                                         int32_t batch, int32_t max_blocks, int32_t block_size) {
  if (batch < 0 || max_blocks < 0 || block_size <= 0) return NVJ_ERR_BAD_SHAPE;
  if (token_bytes != 4 && token_bytes != 8) return NVJ_ERR_BAD_DTYPE;
  if (batch == 0) return NVJ_OK;
  if (!next_tokens || !input_ids || !positions || !context_lens || !slot_mapping)
    return NVJ_ERR_NULL_POINTER;
  if (max_blocks > 0 && !block_tables) return NVJ_ERR_NULL_POINTER;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((batch + 255) / 256)), block(256);
  const hipError_t rc =
      token_bytes == 8
          ? nvj::launch(advance_decode_kernel<int64_t>, grid, block, s,
                        static_cast<const int64_t*>(next_tokens), input_ids, positions,
                        context_lens, slot_mapping, block_tables, batch, max_blocks, block_size)
          : nvj::launch(advance_decode_kernel<int32_t>, grid, block, s,
                        static_cast<const int32_t*>(next_tokens), input_ids, positions,
                        context_lens, slot_mapping, block_tables, batch, max_blocks, block_size);
  return rc == hipSuccess ? NVJ_OK : NVJ_ERR_LAUNCH;
}

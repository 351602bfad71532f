/*
 * A caller of the C ABI written in plain C (no C++, no torch, no Python in the
 * process): what a host in another language binds through its FFI.  It reads one
 * problem from a file, runs the KV-cache store and the paged decode attention
 * through include/nvj_paged_attn.h on device 0 and writes the results to a
 * second file; the test that drives it compares them with the CPU oracle.
 *
 *   nvj_c_caller <problem file> <result file>
 *
 * Problem file (little endian): 12 int32 {batch, num_heads, num_kv_heads,
 * head_dim, block_size, max_blocks, num_blocks, chunk, dtype, k_new_is_f32, 0,
 * 0}, float32 scale, then the arrays q, k_cache, v_cache (16-bit patterns),
 * block_tables, context_lens, slot_mapping (int32), k_new (16-bit or float32),
 * v_new (16-bit).  Result file: out, k_cache, v_cache (16-bit patterns).
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "nvj_paged_attn.h"

static void die(const char* what, int code) {
  fprintf(stderr, "nvj_c_caller: %s (code %d)\n", what, code);
  exit(1);
}

static void* read_array(FILE* f, size_t bytes) {
  void* p = malloc(bytes ? bytes : 1);
  if (!p || (bytes && fread(p, 1, bytes, f) != bytes)) die("short problem file", 0);
  return p;
}

static void* to_device(const void* host, size_t bytes) {
  void* d = NULL;
  if (hipMalloc(&d, bytes ? bytes : 16) != hipSuccess) die("hipMalloc failed", 0);
  if (host && bytes && hipMemcpy(d, host, bytes, hipMemcpyHostToDevice) != hipSuccess)
    die("hipMemcpy to the device failed", 0);
  return d;
}

int main(int argc, char** argv) {
  if (argc != 3) die("usage: nvj_c_caller <problem file> <result file>", 0);
  if (nvj_abi_version() != NVJ_ABI_VERSION) die("library and header disagree on the ABI", 0);
  FILE* f = fopen(argv[1], "rb");
  if (!f) die("cannot open the problem file", 0);
  int32_t h[12];
  float scale;
  if (fread(h, sizeof(int32_t), 12, f) != 12 || fread(&scale, sizeof(float), 1, f) != 1)
    die("short header", 0);
  const int32_t batch = h[0], hq = h[1], hkv = h[2], d = h[3], bs = h[4], mb = h[5], nb = h[6],
                chunk = h[7], dtype = h[8], k_f32 = h[9];
  const size_t q_bytes = (size_t)batch * hq * d * 2;
  const size_t cache_bytes = (size_t)nb * bs * hkv * d * 2;
  const size_t new_rows = (size_t)batch * hkv * d;
  void* q = read_array(f, q_bytes);
  void* kc = read_array(f, cache_bytes);
  void* vc = read_array(f, cache_bytes);
  void* bt = read_array(f, (size_t)batch * mb * 4);
  void* ctx = read_array(f, (size_t)batch * 4);
  void* slots = read_array(f, (size_t)batch * 4);
  void* k_new = read_array(f, new_rows * (k_f32 ? 4 : 2));
  void* v_new = read_array(f, new_rows * 2);
  fclose(f);

  if (hipSetDevice(0) != hipSuccess) die("no GPU", 0);
  hipStream_t stream;
  if (hipStreamCreate(&stream) != hipSuccess) die("hipStreamCreate failed", 0);
  void* dq = to_device(q, q_bytes);
  void* dkc = to_device(kc, cache_bytes);
  void* dvc = to_device(vc, cache_bytes);
  void* dbt = to_device(bt, (size_t)batch * mb * 4);
  void* dctx = to_device(ctx, (size_t)batch * 4);
  void* dslots = to_device(slots, (size_t)batch * 4);
  void* dk_new = to_device(k_new, new_rows * (k_f32 ? 4 : 2));
  void* dv_new = to_device(v_new, new_rows * 2);
  void* dout = to_device(NULL, q_bytes);
  const size_t ws_bytes = nvj_paged_decode_workspace_bytes(batch, hq, d, mb, bs, hkv, chunk);
  void* dws = to_device(NULL, ws_bytes);

  /* store the new rows, then attend over the cache that now holds them */
  int rc = nvj_store_kvcache_launch(stream, dk_new, dv_new, dkc, dvc, (const int32_t*)dslots,
                                    batch, hkv, d, (int64_t)nb * bs,
                                    k_f32 ? NVJ_DTYPE_F32 : dtype, dtype, dtype);
  if (rc != NVJ_OK) die(nvj_error_string(rc), rc);
  rc = nvj_paged_decode_launch(stream, dq, dkc, dvc, (const int32_t*)dbt, (const int32_t*)dctx,
                               dout, dws, ws_bytes, batch, hq, hkv, d, bs, mb, nb, scale, chunk,
                               dtype);
  if (rc != NVJ_OK) die(nvj_error_string(rc), rc);
  if (hipStreamSynchronize(stream) != hipSuccess) die("the launches failed on the device", 0);

  void* out = malloc(q_bytes ? q_bytes : 1);
  if (hipMemcpy(out, dout, q_bytes, hipMemcpyDeviceToHost) != hipSuccess ||
      hipMemcpy(kc, dkc, cache_bytes, hipMemcpyDeviceToHost) != hipSuccess ||
      hipMemcpy(vc, dvc, cache_bytes, hipMemcpyDeviceToHost) != hipSuccess)
    die("hipMemcpy to the host failed", 0);
  f = fopen(argv[2], "wb");
  if (!f) die("cannot open the result file", 0);
  if (fwrite(out, 1, q_bytes, f) != q_bytes || fwrite(kc, 1, cache_bytes, f) != cache_bytes ||
      fwrite(vc, 1, cache_bytes, f) != cache_bytes)
    die("short write", 0);
  fclose(f);
  printf("nvj_c_caller: ok (batch %d, workspace %zu bytes)\n", batch, ws_bytes);
  return 0;
}

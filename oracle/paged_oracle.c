/*
 * C restatement of the reference's KV-cache store and paged decode attention.
 * TEST INFRASTRUCTURE ONLY: it is the checker for tests/, for
 * __graft_entry__.smoke() and the cpu_baseline leg of bench.py; the product
 * library never links or calls it.
 *
 * Same arithmetic as oracle/paged_attention_oracle.py (fp32, two passes over
 * the live positions of a sequence), with OpenMP over (sequence, kv head) so
 * that it can stand as the host-core baseline.  Paths cited are relative to
 * the reference checkout.  Pinned by tests/test_oracle_pinning.py against the
 * NumPy restatement and, through it, against the fp64 brute force and the
 * closed forms.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define CLONES __attribute__((target_clones("avx2,fma", "default")))

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round to nearest even, NaN kept quiet (astype(bfloat16), layers/attention.py:70-71) */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  return (uint16_t)((u + (((u >> 16) & 1u) + 0x7FFFu)) >> 16);
}

/* IEEE half <-> f32; rounding to nearest even, overflow to inf, NaN kept quiet */
static inline float f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else {                       /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7F800000u | (man << 13);
  } else {
    u = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu));   /* NaN */
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);                         /* >= 65536: inf */
  if (a < 0x38800000u) {           /* below the smallest normal half: subnormal or zero */
    if (a < 0x33000000u) return sign;                      /* < 2^-25 rounds to zero */
    const int shift = 126 - (int)(a >> 23);                /* 14 .. 24 */
    const uint32_t man = (a & 0x7FFFFFu) | 0x800000u;
    const uint32_t q = man >> shift, rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    return (uint16_t)(sign | (q + (rem > half || (rem == half && (q & 1u)))));
  }
  const uint32_t r = a + 0xFFFu + ((a >> 13) & 1u);        /* round the 13 dropped bits */
  if (r >= 0x47800000u) return (uint16_t)(sign | 0x7C00u);
  return (uint16_t)(sign | ((r - 0x38000000u) >> 13));
}

/* element codec by cache dtype: 0 = bf16, 2 = IEEE half (the codes of the C ABI) */
static inline float elem_to_f32(uint16_t b, int f16) { return f16 ? f16_to_f32(b) : bf16_to_f32(b); }
static inline uint16_t f32_to_elem(float f, int f16) { return f16 ? f32_to_f16(f) : f32_to_bf16(f); }

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/*
 * store_kv_to_cache (layers/attention.py:42-77).  key/value are f32 when
 * *_is_f32 is non-zero, bf16 bits otherwise.  negative_mode 0 = the code's
 * behaviour (negative slot -> row 0, :64-67), 1 = skip (docstring, :57-58).
 * Slots >= num_slots are dropped (:74).  Later tokens overwrite earlier ones.
 */
void oracle_store_kvcache(const void* key, const void* value, uint16_t* k_cache,
                          uint16_t* v_cache, const int32_t* slot_mapping, int num_tokens,
                          int row_elems, int64_t num_slots, int k_is_f32, int v_is_f32,
                          int negative_mode, int cache_is_f16) {
  for (int t = 0; t < num_tokens; ++t) {
    int64_t slot = slot_mapping[t];
    if (slot < 0) {
      if (negative_mode == 1) continue;
      slot = 0;
    }
    if (slot >= num_slots) continue;
    uint16_t* kd = k_cache + slot * row_elems;
    uint16_t* vd = v_cache + slot * row_elems;
    for (int e = 0; e < row_elems; ++e) {
      kd[e] = k_is_f32 ? f32_to_elem(((const float*)key)[(int64_t)t * row_elems + e], cache_is_f16)
                       : ((const uint16_t*)key)[(int64_t)t * row_elems + e];
      vd[e] = v_is_f32 ? f32_to_elem(((const float*)value)[(int64_t)t * row_elems + e], cache_is_f16)
                       : ((const uint16_t*)value)[(int64_t)t * row_elems + e];
    }
  }
}

/* one (sequence, kv head): scores, softmax, weighted sum for its G query heads */
CLONES static void decode_one(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                              const int32_t* table, int ctx, float* out, float* scores, int G,
                              int D, int bs, int Hkv, int NB, int kvh, float scale, int f16) {
  const int64_t row = (int64_t)Hkv * D;
  float qf[16 * 256];
  for (int g = 0; g < G; ++g)
    for (int d = 0; d < D; ++d) qf[g * D + d] = elem_to_f32(q[g * D + d], f16);
  /* scores = (q . k) * scale   (layers/pallas_attention.py:208-214) */
  for (int s = 0; s < ctx; ++s) {
    int page = table[s / bs];
    page = page < 0 ? 0 : (page > NB - 1 ? NB - 1 : page);          /* :185 */
    const uint16_t* kr = k_cache + ((int64_t)page * bs + s % bs) * row + (int64_t)kvh * D;
    float kf[256];
    if (f16) for (int d = 0; d < D; ++d) kf[d] = f16_to_f32(kr[d]);
    else for (int d = 0; d < D; ++d) kf[d] = bf16_to_f32(kr[d]);
    for (int g = 0; g < G; ++g) {
      float acc = 0.f;
      for (int d = 0; d < D; ++d) acc += qf[g * D + d] * kf[d];
      scores[(int64_t)g * ctx + s] = acc * scale;
    }
  }
  /* softmax over live positions; masked ones weigh exactly 0 (:216-227) */
  float inv[16];
  for (int g = 0; g < G; ++g) {
    float* sc = scores + (int64_t)g * ctx;
    float mx = -1e9f;
    for (int s = 0; s < ctx; ++s) mx = sc[s] > mx ? sc[s] : mx;
    float sum = 0.f;
    for (int s = 0; s < ctx; ++s) {
      sc[s] = expf(sc[s] - mx);
      sum += sc[s];
    }
    inv[g] = 1.0f / (sum + 1e-9f);
    for (int d = 0; d < D; ++d) out[g * D + d] = 0.f;
  }
  /* out = sum_s w[s] * v[s]   (:231-236) */
  for (int s = 0; s < ctx; ++s) {
    int page = table[s / bs];
    page = page < 0 ? 0 : (page > NB - 1 ? NB - 1 : page);
    const uint16_t* vr = v_cache + ((int64_t)page * bs + s % bs) * row + (int64_t)kvh * D;
    float vf[256];
    if (f16) for (int d = 0; d < D; ++d) vf[d] = f16_to_f32(vr[d]);
    else for (int d = 0; d < D; ++d) vf[d] = bf16_to_f32(vr[d]);
    for (int g = 0; g < G; ++g) {
      const float w = scores[(int64_t)g * ctx + s] * inv[g];
      for (int d = 0; d < D; ++d) out[g * D + d] += w * vf[d];
    }
  }
}

/*
 * paged_decode_attention_vectorized (layers/pallas_attention.py:146-238).
 * out_f32 (may be NULL) receives the unrounded result, out_bf16 (may be NULL)
 * the result rounded like .astype(q.dtype) (:238).  Returns 0, or -1 on
 * unsupported sizes (G > 16, D > 256) or allocation failure.  elem_f16 != 0: q,
 * the caches and the rounded output are IEEE half instead of bf16.
 */
int oracle_paged_decode(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                        const int32_t* block_tables, const int32_t* context_lens,
                        float* out_f32, uint16_t* out_bf16, int B, int Hq, int Hkv, int D,
                        int bs, int MB, int NB, float scale, int elem_f16) {
  if (Hkv <= 0 || Hq % Hkv != 0) return -1;
  const int G = Hq / Hkv;
  if (G > 16 || D > 256) return -1;
  int failed = 0;
#pragma omp parallel
  {
    float* scores = NULL;
    int cap = 0;
    float o[16 * 256];
#pragma omp for collapse(2) schedule(dynamic, 1)
    for (int b = 0; b < B; ++b) {
      for (int kvh = 0; kvh < Hkv; ++kvh) {
        int ctx = context_lens[b];
        if (ctx > MB * bs) ctx = MB * bs;
        if (ctx < 0) ctx = 0;
        if (ctx > cap) {
          free(scores);
          scores = (float*)malloc((size_t)G * ctx * sizeof(float));
          cap = scores ? ctx : 0;
          if (!scores) { failed = 1; continue; }
        }
        if (ctx == 0) {
          memset(o, 0, sizeof(float) * G * D);                       /* 0 / (0 + 1e-9) */
        } else {
          decode_one(q + ((int64_t)b * Hq + (int64_t)kvh * G) * D, k_cache, v_cache,
                     block_tables + (int64_t)b * MB, ctx, o, scores, G, D, bs, Hkv, NB, kvh, scale,
                     elem_f16);
        }
        for (int g = 0; g < G; ++g)
          for (int d = 0; d < D; ++d) {
            const int64_t idx = ((int64_t)b * Hq + (int64_t)kvh * G + g) * D + d;
            if (out_f32) out_f32[idx] = o[g * D + d];
            if (out_bf16) out_bf16[idx] = f32_to_elem(o[g * D + d], elem_f16);
          }
      }
    }
    free(scores);
  }
  return failed ? -1 : 0;
}

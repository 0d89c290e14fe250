/*
 * paged_attention_oracle.c -- CPU restatement of the reference's paged-attention path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP kernels: it may be
 * called from tests/, from __graft_entry__.smoke() and from the cpu_baseline leg of
 * bench.py, never from the product path.
 *
 * What it restates (paths relative to the reference root):
 *   store_kv_cache            mini-sglang-mlx-kernel/csrc/store_kv_cache.metal:19-30
 *   paged_prefill_attention   mini-sglang-mlx-kernel/csrc/paged_prefill_attention.metal
 *                               mask predicate :339-347, kv limit :447-450,
 *                               all-masked row -> 0 :366-371, 546-554, 627-630
 *   paged_decode_attention    mini-sglang-mlx-kernel/csrc/paged_decode_attention.metal
 *                               split geometry :356-363, per-split partial + LSE :481-505,
 *                               merge :554-584
 *   kv head of a q head       paged_prefill_attention.metal:422-423 (kvh = h / (n_q/n_kv))
 *
 * Arithmetic: inputs are bf16 bit patterns (uint16); they are widened exactly and
 * everything is evaluated in `acc_t` (double by default, float when compiled with
 * -DORACLE_ACC_FLOAT for the timed CPU baseline).  The result is returned both as
 * acc->float and rounded once to bf16 (round-to-nearest-even), the dtype of q.
 *
 * Parity status: the reference kernels are Metal-only and cannot run here, and MLX
 * (whose CPU SDPA the reference's own scripts compare against) is not installed.
 * Pinned by: the closed-form mask cases of test_and_bench/test_paged_prefill_attention_masks.py
 * (all seven), the row-loop equality of test_and_bench/store_kv_cache.py, an independent
 * numpy float64 softmax-attention on small random inputs, and the invariants in
 * tests/test_oracle_*.py.  Bit-level rounding of the Metal kernels (fp32 P into PV,
 * fast::exp2) is NOT reproduced: parity against MLX-CPU SDPA itself is unpinned.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef ORACLE_ACC_FLOAT
typedef float acc_t;
#define ACC_EXP expf
#define ACC_LOG logf
#else
typedef double acc_t;
#define ACC_EXP exp
#define ACC_LOG log
#endif

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = ((uint32_t)b) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even, NaN kept quiet */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

int oracle_acc_bytes(void) { return (int)sizeof(acc_t); }

/* ------------------------------------------------------------------------- */
/* store_kv_cache.metal:19-30 -- row scatter, bit copy                        */
/* strides in elements; row_elems = num_kv_heads * head_dim                   */
/* ------------------------------------------------------------------------- */
void oracle_store_kv_cache(void* k_cache, void* v_cache, const int32_t* indices,
                           const void* k, const void* v, int64_t length,
                           int64_t row_elems, int64_t k_cache_stride0,
                           int64_t v_cache_stride0, int64_t k_stride0,
                           int64_t v_stride0, int32_t elem_bytes) {
  const size_t row_bytes = (size_t)row_elems * (size_t)elem_bytes;
  for (int64_t r = 0; r < length; ++r) {
    const int64_t slot = indices[r];
    memcpy((char*)k_cache + (size_t)slot * k_cache_stride0 * elem_bytes,
           (const char*)k + (size_t)r * k_stride0 * elem_bytes, row_bytes);
    memcpy((char*)v_cache + (size_t)slot * v_cache_stride0 * elem_bytes,
           (const char*)v + (size_t)r * v_stride0 * elem_bytes, row_bytes);
  }
}

/* ------------------------------------------------------------------------- */
/* One query row against keys [j_lo, j_hi) of a request, with the reference's */
/* visibility predicate.  Returns the un-normalised accumulator, running max  */
/* and sum (natural-log domain), so the same routine serves the one-pass      */
/* prefill form and the split form of decode.                                 */
/* ------------------------------------------------------------------------- */
static void attend_range(const uint16_t* qrow, const uint16_t* k_cache,
                         const uint16_t* v_cache, const int32_t* kv_idx,
                         int64_t j_lo, int64_t j_hi, int64_t kvh, int64_t d,
                         int64_t k_stride0, int64_t v_stride0, acc_t sm_scale,
                         int64_t qpos, int is_cross, int64_t window,
                         acc_t* acc /* d */, acc_t* out_max, acc_t* out_sum) {
  acc_t m = -INFINITY, s = 0;
  for (int64_t c = 0; c < d; ++c) acc[c] = 0;
  for (int64_t j = j_lo; j < j_hi; ++j) {
    /* paged_prefill_attention.metal:339-347 */
    const int in_causal = is_cross || (j <= qpos);
    const int in_window = (window == 0) || (j >= qpos - window + 1);
    if (!(in_causal && in_window)) continue;
    const int64_t slot = kv_idx[j];
    const uint16_t* krow = k_cache + slot * k_stride0 + kvh * d;
    const uint16_t* vrow = v_cache + slot * v_stride0 + kvh * d;
    acc_t dot = 0;
    for (int64_t c = 0; c < d; ++c)
      dot += (acc_t)bf16_to_f32(qrow[c]) * (acc_t)bf16_to_f32(krow[c]);
    const acc_t sc = dot * sm_scale;
    if (sc > m) {
      const acc_t f = (m == -INFINITY) ? 0 : ACC_EXP(m - sc);
      for (int64_t c = 0; c < d; ++c) acc[c] *= f;
      s *= f;
      m = sc;
    }
    const acc_t p = ACC_EXP(sc - m);
    s += p;
    for (int64_t c = 0; c < d; ++c) acc[c] += p * (acc_t)bf16_to_f32(vrow[c]);
  }
  *out_max = m;
  *out_sum = s;
}

/* ------------------------------------------------------------------------- */
/* paged_prefill_attention (paged_prefill_attention.metal:382-640)            */
/*   q   (total_q, n_q, d) bf16 bits;  pools (slots, n_kv, d) with stride0    */
/*   out_f32 / out_bf16: (total_q, n_q, d); either may be NULL                */
/* Rows i >= max_len_extend of a request are left untouched, as the           */
/* reference's grid never reaches them (paged_prefill_attention.cpp:152-159). */
/* ------------------------------------------------------------------------- */
void oracle_paged_prefill_attention(
    const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
    const int32_t* qo_indptr, const int32_t* kv_indptr, const int32_t* kv_indices,
    const int32_t* prefix_lens, float* out_f32, uint16_t* out_bf16, int64_t batch,
    int64_t n_q, int64_t n_kv, int64_t d, int64_t k_stride0, int64_t v_stride0,
    float sm_scale, int64_t max_len_extend, int32_t is_cross, int64_t window) {
  const int64_t group = n_q / n_kv;
#pragma omp parallel
  {
    acc_t* acc = (acc_t*)malloc(sizeof(acc_t) * (size_t)d);
    for (int64_t b = 0; b < batch; ++b) {
      const int64_t q0 = qo_indptr[b];
      int64_t qn = qo_indptr[b + 1] - q0;
      if (qn > max_len_extend) qn = max_len_extend;
      const int64_t k0 = kv_indptr[b];
      const int64_t kn = kv_indptr[b + 1] - k0;
      const int64_t prefix = prefix_lens[b];
#pragma omp for collapse(2) schedule(dynamic, 8) nowait
      for (int64_t i = 0; i < qn; ++i) {
        for (int64_t h = 0; h < n_q; ++h) {
          const int64_t qpos = prefix + i;
          /* paged_prefill_attention.metal:447-450: keys beyond the causal limit
             are never visited; the predicate alone already excludes them. */
          acc_t m, s;
          attend_range(q + ((q0 + i) * n_q + h) * d, k_cache, v_cache,
                       kv_indices + k0, 0, kn, h / group, d, k_stride0, v_stride0,
                       (acc_t)sm_scale, qpos, is_cross, window, acc, &m, &s);
          const acc_t inv = (s > 0) ? (acc_t)1 / s : 0; /* :627-630 */
          for (int64_t c = 0; c < d; ++c) {
            const float o = (float)(acc[c] * inv);
            const int64_t off = ((q0 + i) * n_q + h) * d + c;
            if (out_f32) out_f32[off] = o;
            if (out_bf16) out_bf16[off] = f32_to_bf16(o);
          }
        }
      }
    }
    free(acc);
  }
}

/* split geometry, paged_decode_attention.metal:356-360 */
int64_t oracle_decode_kv_len_per_split(int64_t seq_len, int64_t kv_splits) {
  const int64_t min_block = 32;
  return ((seq_len + kv_splits - 1) / kv_splits + min_block - 1) / min_block * min_block;
}

/* ------------------------------------------------------------------------- */
/* paged_decode_attention as the reference computes it: stage 1 writes, per   */
/* (request, q head, split), the NORMALISED partial and lse = max + ln(sum)   */
/* (paged_decode_attention.metal:481-505); stage 2 merges the non-empty       */
/* splits in order (:554-584).  att_out (batch, n_q, max_kv_splits, d) and    */
/* att_lse (batch, n_q, max_kv_splits) are optional outputs (NULL to skip).   */
/* A request with no tokens gets zeros (the reference leaves it unwritten).   */
/* ------------------------------------------------------------------------- */
void oracle_paged_decode_attention(
    const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
    const int32_t* kv_indptr, const int32_t* kv_indices, const int32_t* num_kv_splits,
    float* out_f32, uint16_t* out_bf16, float* att_out, float* att_lse, int64_t batch,
    int64_t n_q, int64_t n_kv, int64_t d, int64_t k_stride0, int64_t v_stride0,
    float sm_scale, int64_t max_kv_splits) {
  const int64_t group = n_q / n_kv;
#pragma omp parallel
  {
    acc_t* part = (acc_t*)malloc(sizeof(acc_t) * (size_t)d);
    acc_t* acc = (acc_t*)malloc(sizeof(acc_t) * (size_t)d);
#pragma omp for collapse(2) schedule(dynamic, 1)
    for (int64_t b = 0; b < batch; ++b) {
      for (int64_t h = 0; h < n_q; ++h) {
        const int64_t k0 = kv_indptr[b];
        const int64_t len = kv_indptr[b + 1] - k0;
        const int64_t off = (b * n_q + h) * d;
        if (len <= 0) {
          for (int64_t c = 0; c < d; ++c) {
            if (out_f32) out_f32[off + c] = 0.0f;
            if (out_bf16) out_bf16[off + c] = 0;
          }
          continue;
        }
        int64_t splits = num_kv_splits[b];
        if (splits < 1) splits = 1;
        if (splits > max_kv_splits) splits = max_kv_splits;
        const int64_t per = oracle_decode_kv_len_per_split(len, splits);
        acc_t e_max = -INFINITY, e_sum = 0;
        for (int64_t c = 0; c < d; ++c) acc[c] = 0;
        for (int64_t sp = 0; sp < splits; ++sp) {
          const int64_t lo = per * sp;
          int64_t hi = lo + per;
          if (hi > len) hi = len;
          if (lo >= hi) break; /* :363 and :557 */
          acc_t m, s;
          /* decode: every key of the request is visible (qpos = len-1, causal) */
          attend_range(q + (b * n_q + h) * d, k_cache, v_cache, kv_indices + k0, lo, hi,
                       h / group, d, k_stride0, v_stride0, (acc_t)sm_scale, len - 1, 0,
                       0, part, &m, &s);
          const acc_t inv = (s > 0) ? (acc_t)1 / s : 0;
          const acc_t lse = m + ACC_LOG(s); /* :502 */
          if (att_lse) att_lse[(b * n_q + h) * max_kv_splits + sp] = (float)lse;
          for (int64_t c = 0; c < d; ++c) {
            part[c] *= inv;
            if (att_out)
              att_out[((b * n_q + h) * max_kv_splits + sp) * d + c] = (float)part[c];
          }
          /* :562-575 */
          const acc_t new_max = (lse > e_max) ? lse : e_max;
          const acc_t old_scale = (e_max == -INFINITY) ? 0 : ACC_EXP(e_max - new_max);
          const acc_t new_scale = ACC_EXP(lse - new_max);
          for (int64_t c = 0; c < d; ++c) acc[c] = acc[c] * old_scale + new_scale * part[c];
          e_sum = e_sum * old_scale + new_scale;
          e_max = new_max;
        }
        const acc_t inv = (e_sum > 0) ? (acc_t)1 / e_sum : 0;
        for (int64_t c = 0; c < d; ++c) {
          const float o = (float)(acc[c] * inv);
          if (out_f32) out_f32[off + c] = o;
          if (out_bf16) out_bf16[off + c] = f32_to_bf16(o);
        }
      }
    }
    free(part);
    free(acc);
  }
}

/* bf16 helpers exported for the tests (rounding must match torch's) */
void oracle_f32_to_bf16(const float* src, uint16_t* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_bf16(src[i]);
}
void oracle_bf16_to_f32(const uint16_t* src, float* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(src[i]);
}

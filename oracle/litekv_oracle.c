/*
 * litekv_oracle.c -- CPU restatement of the reference's paged-KV attention
 * path, in plain C.
 *
 * THIS IS TEST INFRASTRUCTURE. It is the checker the HIP kernels are compared
 * with (tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py);
 * the product (llama_lite_npu_amd/) never links, imports or calls it.
 *
 * Each function cites the reference file:line (relative to the reference
 * checkout) whose arithmetic it restates. Data is fp16 stored as uint16_t;
 * attention accumulates in fp32, or in fp64 when `wide` is non-zero, and
 * returns unrounded fp32 so callers can apply their own tolerance.
 *
 * What pins each function (see tests/test_oracle.py):
 *   oracle_kv_append, oracle_page_gather  closed form (index assignment),
 *       sentinel-fill invariants, gather(scatter) == identity, and the
 *       PyTorch index-assignment restatement in oracle/cpu_ref.py
 *   oracle_paged_decode, oracle_paged_prefill, oracle_varlen_prefill
 *       brute-force Python loops on tiny inputs, the PyTorch
 *       matmul/softmax/scaled_dot_product_attention restatement in
 *       oracle/cpu_ref.py, and closed forms (one token => out == v,
 *       equal keys => out == mean(V), chunked == rows of the full result)
 *   oracle_decode_partitioned, oracle_lse_merge  equality with the one-pass
 *       softmax for any partition size; associativity
 * The reference ships no golden vectors for these numerics (its kernel tests
 * are allclose-to-inline-torch scripts that need an NPU), so numeric parity
 * with the Triton kernels themselves is "parity unpinned"; the integer
 * examples its tests do hold (slot = page * page_size + offset tables) are
 * checked in tests/test_host_paging.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: renormalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* Exposed so tests can pin the conversion against numpy's float16. */
float oracle_half_to_float(uint16_t h) { return half_to_float(h); }

/*
 * KV_Buffer[Select_Index[i], :, :] = KV_Values[i, :, :]
 * (lite_llama/kernels/update_kv_buffer.py:47-56; torch form :104-105).
 * row_elems = 2 * Hkv * D. Slots outside [0, num_slots) are skipped.
 */
void oracle_kv_append(const uint16_t *kv_values, const int32_t *select_index, uint16_t *kv_buffer,
                      int64_t num_tokens, int64_t row_elems, int64_t num_slots) {
  for (int64_t t = 0; t < num_tokens; ++t) {
    int64_t slot = select_index[t];
    if (slot < 0 || slot >= num_slots) continue;
    memcpy(kv_buffer + slot * row_elems, kv_values + t * row_elems, (size_t)row_elems * 2);
  }
}

/*
 * dst[dst_ids[i]] = src[src_ids[i]] over whole pages (dst_ids NULL: page i).
 * No counterpart in the reference (its allocator never moves KV,
 * lite_llama/executor/paged_attention.py:1-11); closed form only.
 * Moves are applied as if all sources were read before any destination is
 * written (sources are buffered), matching the kernel's contract that a
 * destination is never another move's source.
 */
void oracle_page_gather(const uint16_t *src_pool, uint16_t *dst_pool, const int32_t *src_ids,
                        const int32_t *dst_ids, int64_t n, int64_t page_elems,
                        int64_t num_src_pages, int64_t num_dst_pages) {
  uint16_t *tmp = (uint16_t *)malloc((size_t)(n > 0 ? n : 1) * (size_t)page_elems * 2);
  for (int64_t i = 0; i < n; ++i) {
    int64_t sp = src_ids[i];
    if (sp < 0 || sp >= num_src_pages) continue;
    memcpy(tmp + i * page_elems, src_pool + sp * page_elems, (size_t)page_elems * 2);
  }
  for (int64_t i = 0; i < n; ++i) {
    int64_t sp = src_ids[i];
    int64_t dp = dst_ids ? dst_ids[i] : i;
    if (sp < 0 || sp >= num_src_pages || dp < 0 || dp >= num_dst_pages) continue;
    memcpy(dst_pool + dp * page_elems, tmp + i * page_elems, (size_t)page_elems * 2);
  }
  free(tmp);
}

/* slot of logical token t: page table lookup, slot = page * PS + t % PS
 * (lite_llama/executor/paged_attention.py:141-146, 347-354). */
static int64_t slot_of(const int32_t *table_row, int64_t t, int ps) {
  return (int64_t)table_row[t / ps] * ps + (t % ps);
}

/*
 * One (query row, head) of softmax(q . K^T * scale) V over keys [0, n_keys)
 * addressed by key_row(t). This is the arithmetic of
 * lite_llama/kernels/paged_chunk_flashattention.py:203-221 (fp32 scores,
 * natural softmax, GQA map head // groups) with probabilities kept wide
 * rather than cast to fp16, and equally of
 * lite_llama/kernels/flashdecoding.py:348-358.
 */
static void attend_row(const uint16_t *qrow, int d, int64_t n_keys, const uint16_t *k0,
                       const uint16_t *v0, const int64_t *row_off, double scale, int wide,
                       float *out, float *lse_out) {
  double *sc = (double *)malloc(sizeof(double) * (size_t)(n_keys > 0 ? n_keys : 1));
  double mx = -INFINITY;
  for (int64_t t = 0; t < n_keys; ++t) {
    const uint16_t *kr = k0 + row_off[t];
    double s;
    if (wide) {
      double a = 0.0;
      for (int i = 0; i < d; ++i) a += (double)half_to_float(qrow[i]) * (double)half_to_float(kr[i]);
      s = a * scale;
    } else {
      float a = 0.f;
      for (int i = 0; i < d; ++i) a += half_to_float(qrow[i]) * half_to_float(kr[i]);
      s = (double)(a * (float)scale);
    }
    sc[t] = s;
    if (s > mx) mx = s;
  }
  double den = 0.0;
  for (int64_t t = 0; t < n_keys; ++t) {
    sc[t] = wide ? exp(sc[t] - mx) : (double)expf((float)(sc[t] - mx));
    den += sc[t];
  }
  for (int i = 0; i < d; ++i) {
    double a = 0.0;
    float af = 0.f;
    for (int64_t t = 0; t < n_keys; ++t) {
      float vv = half_to_float(v0[row_off[t] + i]);
      if (wide) a += sc[t] * (double)vv;
      else af += (float)sc[t] * vv;
    }
    out[i] = n_keys > 0 ? (float)((wide ? a : (double)af) / den) : 0.f;
  }
  if (lse_out) *lse_out = (float)(mx + log(den));
  free(sc);
}

/*
 * Paged decode attention: out[b][h] over the seq_lens[b] tokens of sequence b
 * (lite_llama/kernels/flashdecoding.py:294-342 end to end; kv head =
 * h // (Hq / Hkv), :44; tokens gathered through the table, :84-94).
 * pool is [slots][2*Hkv][D]; K heads first, then V heads
 * (lite_llama/models/qwen3.py:68-69). lse (may be NULL) gets log-sum-exp.
 */
void oracle_paged_decode(const uint16_t *q, const uint16_t *pool, const int32_t *block_table,
                         int64_t bt_stride, const int32_t *seq_lens, float *out, float *lse,
                         int batch, int hq, int hkv, int d, int ps, float scale, int wide) {
  const int group = hq / hkv;
  const int64_t row = (int64_t)2 * hkv * d;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int b = 0; b < batch; ++b) {
    for (int h = 0; h < hq; ++h) {
      const int64_t n = seq_lens[b] > 0 ? seq_lens[b] : 0;
      int64_t *off = (int64_t *)malloc(sizeof(int64_t) * (size_t)(n > 0 ? n : 1));
      for (int64_t t = 0; t < n; ++t) off[t] = slot_of(block_table + b * bt_stride, t, ps) * row;
      const int kvh = h / group;
      attend_row(q + ((int64_t)b * hq + h) * d, d, n, pool + (int64_t)kvh * d,
                 pool + (int64_t)(hkv + kvh) * d, off, (double)scale, wide,
                 out + ((int64_t)b * hq + h) * d, lse ? lse + (int64_t)b * hq + h : NULL);
      free(off);
    }
  }
}

/*
 * Stage 2 of flash-decoding: merge n partial outputs by their log-sum-exp,
 * sequentially in index order
 * (lite_llama/kernels/flashdecoding.py:242-267):
 *   m' = max(m, lse_p); acc = e^{m-m'} acc + e^{lse_p-m'} o_p;
 *   den = e^{m-m'} den + e^{lse_p-m'}; out = acc / den.
 */
void oracle_lse_merge(const float *mid_o, const float *mid_lse, int n, int d, float *out) {
  double m = -INFINITY, den = 0.0;
  double *acc = (double *)calloc((size_t)d, sizeof(double));
  for (int p = 0; p < n; ++p) {
    double mn = mid_lse[p] > m ? mid_lse[p] : m;
    double alpha = exp(m - mn);
    double w = exp((double)mid_lse[p] - mn);
    for (int i = 0; i < d; ++i) acc[i] = alpha * acc[i] + w * (double)mid_o[(int64_t)p * d + i];
    den = alpha * den + w;
    m = mn;
  }
  for (int i = 0; i < d; ++i) out[i] = (float)(acc[i] / den);
  free(acc);
}

/*
 * Flash-decoding as the reference structures it: stage 1 over fixed
 * partitions of `partition` tokens producing mid_o = acc / d and
 * lse = m + log d per non-empty partition
 * (lite_llama/kernels/flashdecoding.py:50-62, 96-138), then stage 2.
 * mid_o [B][Hq][P][D], mid_lse [B][Hq][P] with P = max_partitions.
 */
void oracle_decode_partitioned(const uint16_t *q, const uint16_t *pool, const int32_t *block_table,
                               int64_t bt_stride, const int32_t *seq_lens, float *out,
                               float *mid_o, float *mid_lse, int batch, int hq, int hkv, int d,
                               int ps, int partition, int max_partitions, float scale) {
  const int group = hq / hkv;
  const int64_t row = (int64_t)2 * hkv * d;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int b = 0; b < batch; ++b) {
    for (int h = 0; h < hq; ++h) {
      const int64_t n = seq_lens[b] > 0 ? seq_lens[b] : 0;
      const int kvh = h / group;
      const int parts = (int)((n + partition - 1) / partition);
      float *mo = mid_o + ((int64_t)b * hq + h) * max_partitions * d;
      float *ml = mid_lse + ((int64_t)b * hq + h) * max_partitions;
      int64_t *off = (int64_t *)malloc(sizeof(int64_t) * (size_t)partition);
      for (int p = 0; p < parts; ++p) {
        const int64_t t0 = (int64_t)p * partition;
        const int64_t t1 = t0 + partition < n ? t0 + partition : n;
        for (int64_t t = t0; t < t1; ++t)
          off[t - t0] = slot_of(block_table + b * bt_stride, t, ps) * row;
        attend_row(q + ((int64_t)b * hq + h) * d, d, t1 - t0, pool + (int64_t)kvh * d,
                   pool + (int64_t)(hkv + kvh) * d, off, (double)scale, 0, mo + (int64_t)p * d,
                   ml + p);
      }
      free(off);
      if (parts > 0) oracle_lse_merge(mo, ml, parts, d, out + ((int64_t)b * hq + h) * d);
      else memset(out + ((int64_t)b * hq + h) * d, 0, sizeof(float) * (size_t)d);
    }
  }
}

/*
 * Varlen causal prefill over paged KV: query row m of sequence b is at
 * logical position ctx_b + m and sees keys 0 .. ctx_b + m through the table
 * (lite_llama/kernels/paged_chunk_flashattention.py:96-143 kernel,
 * :196-221 torch form). context_lens may be NULL (all zero), which is the
 * no-pad FA2 prefill (lite_llama/kernels/flashattention2_nopad.py:113-131).
 */
void oracle_paged_prefill(const uint16_t *q, const uint16_t *pool, const int32_t *block_table,
                          int64_t bt_stride, const int32_t *cu_q_lens, const int32_t *context_lens,
                          float *out, int batch, int hq, int hkv, int d, int ps, float scale,
                          int wide) {
  const int group = hq / hkv;
  const int64_t row = (int64_t)2 * hkv * d;
  for (int b = 0; b < batch; ++b) {
    const int q0 = cu_q_lens[b];
    const int qn = cu_q_lens[b + 1] - q0;
    const int ctx = context_lens ? context_lens[b] : 0;
    const int64_t total = (int64_t)ctx + qn;
    int64_t *off = (int64_t *)malloc(sizeof(int64_t) * (size_t)(total > 0 ? total : 1));
    for (int64_t t = 0; t < total; ++t) off[t] = slot_of(block_table + b * bt_stride, t, ps) * row;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int m = 0; m < qn; ++m) {
      for (int h = 0; h < hq; ++h) {
        const int kvh = h / group;
        attend_row(q + ((int64_t)(q0 + m) * hq + h) * d, d, (int64_t)ctx + m + 1,
                   pool + (int64_t)kvh * d, pool + (int64_t)(hkv + kvh) * d, off, (double)scale,
                   wide, out + ((int64_t)(q0 + m) * hq + h) * d, NULL);
      }
    }
    free(off);
  }
}

/*
 * Varlen causal prefill over packed contiguous K/V [T][Hkv][D]
 * (lite_llama/kernels/flashattention2_nopad.py:69-163 kernel; torch form
 * :250-274): row m of sequence b sees keys 0 .. m of the same sequence.
 */
void oracle_varlen_prefill(const uint16_t *q, const uint16_t *k, const uint16_t *v,
                           const int32_t *seq_starts, const int32_t *seq_lens, float *out,
                           int batch, int hq, int hkv, int d, float scale, int wide) {
  const int group = hq / hkv;
  const int64_t row = (int64_t)hkv * d;
  for (int b = 0; b < batch; ++b) {
    const int s0 = seq_starts[b];
    const int n = seq_lens[b];
    int64_t *off = (int64_t *)malloc(sizeof(int64_t) * (size_t)(n > 0 ? n : 1));
    for (int t = 0; t < n; ++t) off[t] = (int64_t)(s0 + t) * row;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int m = 0; m < n; ++m) {
      for (int h = 0; h < hq; ++h) {
        const int kvh = h / group;
        attend_row(q + ((int64_t)(s0 + m) * hq + h) * d, d, (int64_t)m + 1, k + (int64_t)kvh * d,
                   v + (int64_t)kvh * d, off, (double)scale, wide,
                   out + ((int64_t)(s0 + m) * hq + h) * d, NULL);
      }
    }
    free(off);
  }
}

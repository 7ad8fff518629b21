/*
 * Scalar C restatement of the reference's algorithms for the hot path — TEST INFRASTRUCTURE ONLY.
 * Nothing in the product links or loads this file; tests/ use it (through oracle/cref.py) as a second,
 * independent checker next to the torch restatement in oracle/golden.py: sequential loops, no library
 * routine, so that a mistake in either shows up as a disagreement.
 *
 * Paths cited are relative to python/triton_dist of Triton-distributed.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- number formats ----------------------------------------------------------------------------- */

/* OCP e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities; S.1111.111 is NaN. */
float oc_e4m3_to_f32(uint8_t b) {
  int sign = b >> 7, e = (b >> 3) & 15, m = b & 7;
  float v;
  if (e == 15 && m == 7) return NAN;
  if (e == 0) v = ldexpf((float)m, -9);          /* subnormal: m/8 * 2^-6 */
  else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return sign ? -v : v;
}

void oc_e4m3_table(float* out256) {
  for (int i = 0; i < 256; ++i) out256[i] = oc_e4m3_to_f32((uint8_t)i);
}

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even, NaN kept quiet */
static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* ---- (b) slice reduction: kernels/amd/gemm_reduce_scatter.py:246-258, fp32 accumulator ------------ */
void oc_reduce_slices_bf16(const uint16_t* c, int64_t stride, int n_slices, int first, int64_t n_elems,
                           uint16_t* out) {
  for (int64_t e = 0; e < n_elems; ++e) {
    float acc = 0.0f;
    for (int i = 0; i < n_slices; ++i) {
      int s = (first + i) % n_slices;
      acc = acc + bf16_to_f32(c[(int64_t)s * stride + e]);
    }
    out[e] = f32_to_bf16(acc);
  }
}

/* ---- (a)/(b) GEMM, C = A[M,K] . B[N,K]^T, double accumulation ------------------------------------ */
void oc_gemm_nt_f64(const float* A, const float* B, double* C, int M, int N, int K) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) acc += (double)A[(int64_t)m * K + k] * (double)B[(int64_t)n * K + k];
      C[(int64_t)m * N + n] = acc;
    }
}

/* fp8 GEMM with per-row / per-column scales (closed form; not in the reference) */
void oc_gemm_e4m3_nt_f64(const uint8_t* A, const uint8_t* B, const float* row_scale, const float* col_scale,
                         double* C, int M, int N, int K) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k)
        acc += (double)oc_e4m3_to_f32(A[(int64_t)m * K + k]) * (double)oc_e4m3_to_f32(B[(int64_t)n * K + k]);
      if (row_scale) acc *= (double)row_scale[m];
      if (col_scale) acc *= (double)col_scale[n];
      C[(int64_t)m * N + n] = acc;
    }
}

/* ---- (c) MoE index construction: test/nvidia/test_all_to_all.py:42-46,49-92,95-96,314 ------------- */
/* Sequential stable counting sort of the flat ids. */
void oc_moe_preprocess(const int32_t* ids, int64_t n, int topk, int G, int32_t* splits, int32_t* cumsum,
                       int32_t* scatter_idx, int32_t* gather_idx, int32_t* topk_idx) {
  for (int g = 0; g < G; ++g) splits[g] = 0;
  for (int64_t i = 0; i < n; ++i) splits[ids[i]] += 1;
  cumsum[0] = 0;
  for (int g = 0; g < G; ++g) cumsum[g + 1] = cumsum[g] + splits[g];
  int32_t* next = (int32_t*)malloc(sizeof(int32_t) * (size_t)G);
  for (int g = 0; g < G; ++g) next[g] = cumsum[g];
  for (int64_t i = 0; i < n; ++i) {
    int32_t p = next[ids[i]]++;
    scatter_idx[i] = p;
    gather_idx[p] = (int32_t)(i / topk);
    if (topk_idx) topk_idx[p] = (int32_t)(i % topk);
  }
  free(next);
}

/* kernels/nvidia/low_latency_all_to_all.py:56-103: rows of destination d → slot d (see golden.dispatch_slots) */
void oc_dispatch_slots(const uint8_t* rows, int64_t row_bytes, const float* scales, const int32_t* gather_idx,
                       const int32_t* cumsum, int W, int Er, int max_m, uint8_t* slot_rows, float* slot_scales,
                       int32_t* splits_out) {
  for (int d = 0; d < W; ++d) {
    int32_t st = cumsum[d * Er], ed = cumsum[(d + 1) * Er];
    for (int32_t p = st; p < ed && p - st < max_m; ++p) {
      int64_t src = gather_idx ? gather_idx[p] : p;
      int64_t dst = (int64_t)d * max_m + (p - st);
      memcpy(slot_rows + dst * row_bytes, rows + src * row_bytes, (size_t)row_bytes);
      if (scales) slot_scales[dst] = scales[src];
    }
  }
  if (splits_out)
    for (int g = 0; g < W * Er; ++g) splits_out[g] = cumsum[g + 1] - cumsum[g];
}

/* kernels/nvidia/low_latency_all_to_all.py:251-270; returns the number of rows written */
int64_t oc_post_process(const uint8_t* slot_rows, int64_t row_bytes, const float* slot_scales, const int32_t* splits,
                        int W, int Er, int max_m, uint8_t* out_rows, float* out_scales) {
  int64_t p = 0;
  for (int d = 0; d < W; ++d) {
    int32_t n = 0;
    for (int j = 0; j < Er; ++j) n += splits[d * Er + j];
    for (int32_t i = 0; i < n; ++i, ++p) {
      int64_t src = (int64_t)d * max_m + i;
      memcpy(out_rows + p * row_bytes, slot_rows + src * row_bytes, (size_t)row_bytes);
      if (slot_scales && out_scales) out_scales[p] = slot_scales[src];
    }
  }
  return p;
}

/* weighted combine: test/nvidia/test_moe_reduce_rs.py:117-122 with the identity expert, e4m3 rows.
 * y[t,h] = sum_k (w[t,k]*scale[p]) * f(row[p,h]), p = scatter_idx[t*topk+k]; fp32, k ascending. */
void oc_combine_e4m3(const uint8_t* sorted_rows, const float* sorted_scales, const int32_t* scatter_idx,
                     const float* topk_w, int64_t T, int topk, int H, float* out) {
  for (int64_t t = 0; t < T; ++t)
    for (int h = 0; h < H; ++h) {
      float acc = 0.0f;
      for (int k = 0; k < topk; ++k) {
        int32_t p = scatter_idx[t * topk + k];
        float coef = topk_w ? topk_w[t * topk + k] : 1.0f;
        if (sorted_scales) coef = coef * sorted_scales[p];
        float prod = coef * oc_e4m3_to_f32(sorted_rows[(int64_t)p * H + h]);
        acc = acc + prod;
      }
      out[t * H + h] = acc;
    }
}

/* ---- (d) decode attention over keys [lo[b], hi[b]) of a paged cache, fp64 --------------------------
 * scores as kernels/nvidia/flash_decode.py:207-221, result = softmax . v and LSE = log sum exp (:235-239).
 * q [B,Hq,D]; caches [pages, page_size, Hkv, D] (float copies of the 16-bit data); table [B, table_stride]. */
void oc_decode_range(const float* q, const float* k_cache, const float* v_cache, const int32_t* table,
                     int64_t table_stride, const int32_t* lo, const int32_t* hi, int B, int Hq, int Hkv, int D,
                     int Dv, int page_size, double scale, double soft_cap, double* out, double* lse) {
  int group = Hq / Hkv;
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < Hq; ++h) {
      int kvh = h / group;
      int n0 = lo[b], n1 = hi[b];
      double* o = out + ((int64_t)b * Hq + h) * Dv;
      for (int d = 0; d < Dv; ++d) o[d] = 0.0;
      if (n1 <= n0) {
        lse[(int64_t)b * Hq + h] = -INFINITY;
        continue;
      }
      double* s = (double*)malloc(sizeof(double) * (size_t)(n1 - n0));
      double mx = -INFINITY;
      for (int n = n0; n < n1; ++n) {
        int64_t page = table[(int64_t)b * table_stride + n / page_size];
        const float* kr = k_cache + ((page * page_size + n % page_size) * Hkv + kvh) * D;
        double acc = 0.0;
        for (int d = 0; d < D; ++d) acc += (double)q[((int64_t)b * Hq + h) * D + d] * (double)kr[d];
        acc *= scale;
        if (soft_cap > 0.0) acc = soft_cap * tanh(acc / soft_cap);
        s[n - n0] = acc;
        if (acc > mx) mx = acc;
      }
      double denom = 0.0;
      for (int n = n0; n < n1; ++n) denom += exp(s[n - n0] - mx);
      for (int n = n0; n < n1; ++n) {
        int64_t page = table[(int64_t)b * table_stride + n / page_size];
        const float* vr = v_cache + ((page * page_size + n % page_size) * Hkv + kvh) * Dv;
        double p = exp(s[n - n0] - mx) / denom;
        for (int d = 0; d < Dv; ++d) o[d] += p * (double)vr[d];
      }
      lse[(int64_t)b * Hq + h] = mx + log(denom);
      free(s);
    }
}

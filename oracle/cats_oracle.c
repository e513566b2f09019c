/*
 * cats_oracle.c -- CPU restatement of the CATS sparse-MLP decode path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests/, __graft_entry__.smoke() and the cpu_baseline leg
 * of bench.py may build, load or call it.  Nothing under cats_amd/ or flash_gemv/ links or imports it.
 *
 * What it restates (paths relative to the CATS tree):
 *   oracle_mlp          the dense-masked CATS MLP, experiments/models/sparse_silu/ugly_utils.py:895-899
 *                         post_act = act_fn(gate_proj(x)); post_act[post_act.abs() <= t] = 0;
 *                         down_proj(post_act * up_proj(x))
 *                       with torch's rounding points: every Linear / SiLU / multiply result is rounded to the
 *                       tensor dtype, sums are formed at higher precision (here: double), the threshold scalar
 *                       is cast to the tensor dtype before the comparison.
 *   oracle_gate         the first line of the above plus flags = |a| > t, flash_gemv/flash_gemv/__init__.py:40-41,46
 *   oracle_sparse_up    z = a * (x . wup[j]) under per-row flags, rows loaded under the union of the flags:
 *                       flash_gemv/flash_gemv/kernels.py:208-254 (wrapper) and :115-177 (masking rules)
 *   oracle_sparse_down  y += sum over union-flagged j of z[b,j] * wdown_t[j,:], kernels.py:416-462
 *   oracle_compact      ascending index list + count of the flagged neurons (the sorted form of what
 *                       flash_gemv/csrc/cuda/fuse_gemv_cmp_cuda.cu:80-84 appends in arrival order)
 *   oracle_get_threshold  ugly_utils.py:236-245
 *   oracle_histogram      torch.histogram over the edges of ugly_utils.py:829-831, as used by :852-860
 *
 * Parity status: the reference holds no golden vectors, known-answer tests or fixtures for this path (its
 * test file prints and saves, it never asserts: flash_gemv/test/test_fuse_gemv_cmp.py:144-550).  Every
 * function here is pinned in tests/test_oracle.py by what the mathematics fixes instead: exhaustive dtype
 * conversion against numpy / torch, SiLU closed-form values, hand-built threshold boundary vectors,
 * all-active == three library GEMVs, all-dead == 0, single-neuron exactness, brute force in float64 on small
 * shapes, and the literal four-line PyTorch formula on CPU tensors.
 *
 * dtype codes: 0 = fp16, 1 = bf16, 2 = fp32 (storage); all arithmetic below is double or float.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---------- dtype conversion (IEEE round-to-nearest-even) ---------- */

static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

uint16_t oracle_f32_to_f16(float f) {
  uint32_t x = f2u(f);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x3ffu));
  if (x >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);
  if (x < 0x38800000u) { /* result is subnormal or zero: round x / 2^-24 to an integer */
    const float scaled = u2f(x) * 16777216.0f; /* exact: power-of-two scaling */
    const float r = nearbyintf(scaled);       /* default rounding mode = nearest even */
    return (uint16_t)(sign | (uint32_t)r);
  }
  uint32_t h = (x - 0x38000000u) >> 13;
  const uint32_t rem = x & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}

float oracle_f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  if (e == 0) {
    const float v = (float)m * (1.0f / 16777216.0f);
    return sign ? -v : v;
  }
  if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

/* round a float through the storage dtype */
float oracle_round(int dtype, float f) {
  if (dtype == 0) return oracle_f16_to_f32(oracle_f32_to_f16(f));
  if (dtype == 1) return oracle_bf16_to_f32(oracle_f32_to_bf16(f));
  return f;
}

static float load_elem(int dtype, const void* p, size_t i) {
  if (dtype == 0) return oracle_f16_to_f32(((const uint16_t*)p)[i]);
  if (dtype == 1) return oracle_bf16_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

static void store_elem(int dtype, void* p, size_t i, float v) {
  if (dtype == 0) ((uint16_t*)p)[i] = oracle_f32_to_f16(v);
  else if (dtype == 1) ((uint16_t*)p)[i] = oracle_f32_to_bf16(v);
  else ((float*)p)[i] = v;
}

/* widen a (rows, cols) dtype matrix to float once, so the inner loops are plain float reads */
static float* widen(int dtype, const void* p, size_t n) {
  float* out = (float*)malloc(n * sizeof(float) + 16);
  for (size_t i = 0; i < n; i++) out[i] = load_elem(dtype, p, i);
  return out;
}

/* ---------- scalar pieces ---------- */

/* SiLU in fp32 on an fp32 argument: x / (1 + exp(-x)); the exp is taken in double and rounded so that the
 * result is the correctly rounded fp32 quotient of correctly rounded operands to within 1 ulp. */
float oracle_silu(float x) { return (float)((double)x / (1.0 + exp(-(double)x))); }

/* Linear output element: double accumulation, one rounding to fp32, one to dtype. */
static float dot_round(int dtype, const float* w, const float* x, int n) {
  double s = 0.0;
  for (int k = 0; k < n; k++) s += (double)w[k] * (double)x[k];
  return oracle_round(dtype, (float)s);
}

/* ---------- the path ---------- */

/* a[b,j] = round(silu(round(x[b,:] . wgate[j,:]))), flag[b,j] = |a| > round(t).  a_out (dtype) / flag_out may be NULL. */
void oracle_gate(const void* x, const void* wgate, int B, int H, int I, int dtype, float t, void* a_out, uint8_t* flag_out) {
  float* xf = widen(dtype, x, (size_t)B * H);
  float* wf = widen(dtype, wgate, (size_t)I * H);
  const float tr = oracle_round(dtype, t);
#pragma omp parallel for schedule(static)
  for (int j = 0; j < I; j++)
    for (int b = 0; b < B; b++) {
      const float g = dot_round(dtype, wf + (size_t)j * H, xf + (size_t)b * H, H);
      const float a = oracle_round(dtype, oracle_silu(g));
      if (a_out) store_elem(dtype, a_out, (size_t)b * I + j, a);
      if (flag_out) flag_out[(size_t)b * I + j] = fabsf(a) > tr ? 1 : 0;
    }
  free(xf);
  free(wf);
}

/* Dense-masked CATS MLP.  wdown is the HF (H, I) layout.  If a_in / flag_in are given (both or neither) the gate
 * stage is skipped and they are used instead -- "identical gate values".  y_out (B,H) dtype; z_out (B,I) dtype
 * optional: the rounded product post_act * up_proj(x). */
void oracle_mlp(const void* x, const void* wgate, const void* wup, const void* wdown, int B, int H, int I, int dtype, float t,
                const void* a_in, const uint8_t* flag_in, void* y_out, void* a_out, uint8_t* flag_out, void* z_out) {
  float* xf = widen(dtype, x, (size_t)B * H);
  float* gf = a_in ? NULL : widen(dtype, wgate, (size_t)I * H);
  float* uf = widen(dtype, wup, (size_t)I * H);
  float* df = widen(dtype, wdown, (size_t)H * I);
  float* z = (float*)calloc((size_t)B * I, sizeof(float));
  const float tr = oracle_round(dtype, t);
#pragma omp parallel for schedule(static)
  for (int j = 0; j < I; j++)
    for (int b = 0; b < B; b++) {
      const size_t o = (size_t)b * I + j;
      float a;
      int live;
      if (a_in) {
        a = load_elem(dtype, a_in, o);
        live = flag_in[o] != 0;
      } else {
        const float g = dot_round(dtype, gf + (size_t)j * H, xf + (size_t)b * H, H);
        a = oracle_round(dtype, oracle_silu(g));
        live = fabsf(a) > tr; /* dead <=> |a| <= t */
      }
      if (a_out) store_elem(dtype, a_out, o, a);
      if (flag_out) flag_out[o] = (uint8_t)live;
      const float post = live ? a : 0.0f;
      const float up = dot_round(dtype, uf + (size_t)j * H, xf + (size_t)b * H, H);
      z[o] = oracle_round(dtype, post * up);
      if (z_out) store_elem(dtype, z_out, o, z[o]);
    }
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int b = 0; b < B; b++) store_elem(dtype, y_out, (size_t)b * H + h, dot_round(dtype, df + (size_t)h * I, z + (size_t)b * I, I));
  free(xf);
  free(gf);
  free(uf);
  free(df);
  free(z);
}

/* Sparse up under flags: out[b,j] = flag[b,j] ? a[b,j] * (x[b,:] . wup[j,:]) : 0, accumulated in double, stored as
 * fp32 (out32 != NULL) or rounded to dtype (out_t != NULL).  The dot product itself is NOT rounded to dtype first
 * (the Triton kernel multiplies the fp32 accumulator by a: kernels.py:183-191). */
void oracle_sparse_up(const void* x, const void* wup, const void* a, const uint8_t* flag, int B, int H, int I, int dtype,
                      float* out32, void* out_t) {
  float* xf = widen(dtype, x, (size_t)B * H);
  float* uf = widen(dtype, wup, (size_t)I * H);
#pragma omp parallel for schedule(static)
  for (int j = 0; j < I; j++)
    for (int b = 0; b < B; b++) {
      const size_t o = (size_t)b * I + j;
      float v = 0.0f;
      if (flag[o]) {
        double s = 0.0;
        for (int k = 0; k < H; k++) s += (double)uf[(size_t)j * H + k] * (double)xf[(size_t)b * H + k];
        v = (float)(s * (double)load_elem(dtype, a, o));
      }
      if (out32) out32[o] = v;
      if (out_t) store_elem(dtype, out_t, o, v);
    }
  free(xf);
  free(uf);
}

/* Sparse down: y32[b,h] += sum over j with any flag[.,j] of z[b,j] * wdown_t[j,h] (double accumulation). */
void oracle_sparse_down(const void* z, const void* wdown_t, const uint8_t* flag, int B, int H, int I, int dtype, float* y32) {
  float* zf = widen(dtype, z, (size_t)B * I);
  float* df = widen(dtype, wdown_t, (size_t)I * H);
  uint8_t* any = (uint8_t*)calloc((size_t)I, 1);
  for (int j = 0; j < I; j++)
    for (int b = 0; b < B; b++) any[j] |= flag[(size_t)b * I + j];
#pragma omp parallel for schedule(static)
  for (int h = 0; h < H; h++)
    for (int b = 0; b < B; b++) {
      double s = 0.0;
      for (int j = 0; j < I; j++)
        if (any[j]) s += (double)zf[(size_t)b * I + j] * (double)df[(size_t)j * H + h];
      y32[(size_t)b * H + h] += (float)s;
    }
  free(zf);
  free(df);
  free(any);
}

/* Ascending indices of the set flags; returns the count. */
int oracle_compact(const uint8_t* flag, int I, int64_t* idx_out) {
  int n = 0;
  for (int j = 0; j < I; j++)
    if (flag[j]) idx_out[n++] = j;
  return n;
}

/* ugly_utils.py:236-245.  counts (nbins) is normalised IN PLACE, as the reference's `histogram_counts /= sum` does;
 * cumulative sum in fp32; index = number of cumsum entries <= sparsity (searchsorted side="right");
 * returns bin_edges[index] (bin_edges has nbins + 1 entries).  *index_out receives the index. */
float oracle_get_threshold(const float* bin_edges, float* counts, int nbins, float sparsity, int* index_out) {
  float total = 0.0f;
  for (int i = 0; i < nbins; i++) total += counts[i];
  for (int i = 0; i < nbins; i++) counts[i] /= total;
  float run = 0.0f;
  int idx = 0;
  for (int i = 0; i < nbins; i++) {
    run += counts[i];
    if (run <= sparsity) idx = i + 1;
  }
  /* cumsum is non-decreasing, so "count of entries <= s" is where a right-sided binary search lands */
  if (index_out) *index_out = idx;
  return bin_edges[idx];
}

/* torch.histogram(values, bins=edges): bin i = [edges[i], edges[i+1]) except the last, which is closed on the right;
 * values outside [edges[0], edges[nbins]] are dropped.  Edges may start / end with -inf / +inf (ugly_utils.py:831). */
void oracle_histogram(const float* values, size_t n, const float* edges, int nbins, float* counts_out) {
  for (int i = 0; i < nbins; i++) counts_out[i] = 0.0f;
  for (size_t q = 0; q < n; q++) {
    const float v = values[q];
    if (!(v >= edges[0] && v <= edges[nbins])) continue;
    int lo = 0, hi = nbins; /* find the last edge <= v */
    while (hi - lo > 1) {
      const int mid = (lo + hi) / 2;
      if (edges[mid] <= v) lo = mid; else hi = mid;
    }
    counts_out[lo] += 1.0f;
  }
}

/*
 * CPU oracle for the SVC (RowMerge) -> vector-sparse SpMM path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement of the
 * reference's algorithms, used only as the checker in tests/, in
 * __graft_entry__.smoke() and as the timed CPU baseline of bench.py.  Nothing
 * in the shipped library links against it or calls it.
 *
 * What each function follows (paths relative to the reference checkout):
 *
 *   oracle_pyset_order      CPython's set insertion/iteration order for small
 *                           non-negative ints (Objects/setobject.c, 3.7-3.12:
 *                           set_add_entry, set_insert_clean, set_table_resize),
 *                           which is what `list(set(a + b))` in
 *                           RowMerge/sparse_matrix_format.py:110 yields.
 *                           Pinned by: the Python runtime's builtin set on
 *                           random inputs (tests/test_oracle.py).
 *   oracle_svc              CVSE.__init__, RowMerge/sparse_matrix_format.py:94-123
 *                           (merge at :110, guard at :109, row pointer at
 *                           :112-113), plus the value packing the consumers
 *                           define (SSpMM/sspmm_test.cpp:90,
 *                           end2end/sspmm_e2e/verify/static_mask.py:36-42).
 *                           Pinned by: golden fixtures written by the reference
 *                           itself (tests/golden), brute-force dense-bitmap
 *                           counts, densify round trip.
 *   oracle_spmm_f32/_f16    host check loop SSpMM/sspmm_test.cpp:75-95 (fp16 ->
 *                           fp32 multiply-add, j ascending); fp16 output is the
 *                           round-to-nearest-even conversion the kernels apply
 *                           (SSpMM/src/spmm_utils/sspmm_output_tile.h:345-352).
 *                           Pinned by: densify + numpy fp64 matmul, identity
 *                           pattern, single-vector outer product.
 *   oracle_sorted_row_swizzle  SortedRowSwizzle, SSpMM/include/bm_test_utils.h:210-225
 *                           (argsort by descending vector-row length; the
 *                           reference's tie order is unspecified, ties here keep
 *                           ascending row index).  Pinned by invariants only.
 *   oracle_sddmm_f16        the sampled product either side of the SpMM in the
 *                           reference's sparse attention block:
 *                           out[j*V+v] = lhs[i*V+v, :] . rhs[col_j, :] for the
 *                           vectors j of vector-row i, fp32 accumulation over the
 *                           feature index ascending, fp16 result
 *                           (end2end/sspmm_e2e/src/cuda/sddmm_kernel.cu:1161-1226,
 *                           check recipe end2end/sspmm_e2e/verify/sddmm.py:36-51).
 *                           Pinned by: numpy fp64 matmul sampled at the pattern.
 *   oracle_softmax_f16      csrSoftmaxKernel_, end2end/sspmm_e2e/src/cuda/
 *                           softmax_kernel.cu:95-165: per dense row, over the
 *                           row's stored entries, exp(x*scaler - max) / sum in
 *                           fp32, fp16 result.  Pinned by: numpy softmax of the
 *                           densified rows with -inf fill (the recipe of
 *                           end2end/sspmm_e2e/verify/softmax.py:36-38).
 *   oracle_minhash_order /  the row reordering that runs ahead of the merge (the
 *   oracle_permute_csr      reference's row_merge_reorder.py step, README.md:36).
 *                           The reference's reorder module is not in its sources,
 *                           so there is nothing of the reference to restate: this
 *                           is the CPU statement of the library's own method
 *                           (stable sort of the rows by two min-hashes of their
 *                           column sets).  PARITY UNPINNED against the reference;
 *                           checked by what the definition fixes (a permutation,
 *                           equal column sets adjacent, keys independent of the
 *                           column order within a row, empty rows last) and by
 *                           numpy's stable argsort on the same keys.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ fp16 */

static float h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
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

/* float -> half, round to nearest even (what __float2half / v_cvt_f16_f32 do). */
static uint16_t f2h_rn(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) { /* inf / nan */
    if (absx > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx < 0x33000001u) { /* < 2^-25 (or exactly 2^-25: ties to even -> 0) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  uint32_t shift;
  uint32_t hexp;
  if (e < -14) { /* subnormal half */
    shift = (uint32_t)(13 + (-14 - e));
    hexp = 0;
  } else {
    shift = 13;
    hexp = (uint32_t)(e + 15);
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  uint32_t out;
  if (hexp == 0) {
    out = q; /* may carry into exponent 1: that is the correct encoding */
  } else {
    out = ((hexp - 1) << 10) + q; /* q has the implicit bit at 0x400 */
  }
  return (uint16_t)(sign | out);
}

float oracle_h2f(uint16_t h) { return h2f(h); }
uint16_t oracle_f2h(float f) { return f2h_rn(f); }

/* ------------------------------------------- CPython set model (int keys) */

#define PYSET_MINSIZE 8
#define LINEAR_PROBES 9
#define PERTURB_SHIFT 5

typedef struct {
  int64_t *tab; /* -1 = unused slot */
  size_t mask;
  size_t fill; /* == used: nothing is ever deleted */
} pyset;

static void pyset_init(pyset *s) {
  s->mask = PYSET_MINSIZE - 1;
  s->fill = 0;
  s->tab = (int64_t *)malloc(PYSET_MINSIZE * sizeof(int64_t));
  for (size_t i = 0; i < PYSET_MINSIZE; ++i) s->tab[i] = -1;
}

static void pyset_free(pyset *s) { free(s->tab); }

/* set_insert_clean: key known absent, no dummies. */
static void pyset_insert_clean(int64_t *tab, size_t mask, int64_t key) {
  size_t perturb = (size_t)key;
  size_t i = (size_t)key & mask;
  for (;;) {
    size_t probes = (i + LINEAR_PROBES <= mask) ? LINEAR_PROBES : 0;
    size_t j = i;
    do {
      if (tab[j] < 0) {
        tab[j] = key;
        return;
      }
      ++j;
    } while (probes--);
    perturb >>= PERTURB_SHIFT;
    i = (i * 5 + 1 + perturb) & mask;
  }
}

static void pyset_resize(pyset *s, size_t minused) {
  size_t newsize = PYSET_MINSIZE;
  while (newsize <= minused) newsize <<= 1;
  int64_t *nt = (int64_t *)malloc(newsize * sizeof(int64_t));
  for (size_t i = 0; i < newsize; ++i) nt[i] = -1;
  for (size_t i = 0; i <= s->mask; ++i)
    if (s->tab[i] >= 0) pyset_insert_clean(nt, newsize - 1, s->tab[i]);
  free(s->tab);
  s->tab = nt;
  s->mask = newsize - 1;
}

/* set_add_entry for a non-negative int key (hash(key) == key). */
static void pyset_add(pyset *s, int64_t key) {
  size_t mask = s->mask;
  size_t perturb = (size_t)key;
  size_t i = (size_t)key & mask;
  for (;;) {
    size_t probes = (i + LINEAR_PROBES <= mask) ? LINEAR_PROBES : 0;
    size_t j = i;
    do {
      if (s->tab[j] < 0) {
        s->tab[j] = key;
        s->fill++;
        if (s->fill * 5 >= mask * 3) pyset_resize(s, s->fill > 50000 ? s->fill * 2 : s->fill * 4);
        return;
      }
      if (s->tab[j] == key) return;
      ++j;
    } while (probes--);
    perturb >>= PERTURB_SHIFT;
    i = (i * 5 + 1 + perturb) & mask;
  }
}

/* list(set(keys[0..n))) -> out; returns the number of distinct keys. */
int64_t oracle_pyset_order(const int32_t *keys, int64_t n, int32_t *out) {
  pyset s;
  pyset_init(&s);
  for (int64_t i = 0; i < n; ++i) pyset_add(&s, keys[i]);
  int64_t m = 0;
  for (size_t i = 0; i <= s.mask; ++i)
    if (s.tab[i] >= 0) out[m++] = (int32_t)s.tab[i];
  pyset_free(&s);
  return m;
}

/* ------------------------------------------------------------------- SVC */

static int cmp_i32(const void *a, const void *b) {
  int32_t x = *(const int32_t *)a, y = *(const int32_t *)b;
  return (x > y) - (x < y);
}

/*
 * RowMerge.  order: 0 = CPython set order (bit-exact with the reference's
 * output files), 1 = ascending.
 *   vec_row_ptr[m_vec+1]  always written.
 *   vec_col  (nullable)   capacity >= nnz entries.
 *   vec_val  (nullable)   capacity >= nnz*V halfs, zero filled then scattered;
 *                         needs csr_val.
 * Returns nvec, or -1 on bad arguments.
 */
int64_t oracle_svc(int32_t M, int32_t K, int32_t V, const int32_t *row_ptr, const int32_t *col_ind,
                   const uint16_t *csr_val, int32_t order, int32_t *vec_row_ptr, int32_t *vec_col,
                   uint16_t *vec_val) {
  if (M < 0 || K < 0 || V <= 0 || !row_ptr || !vec_row_ptr) return -1;
  int32_t m_vec = (M + V - 1) / V;
  int64_t nvec = 0;
  vec_row_ptr[0] = 0;
  int64_t cap = 16;
  int32_t *cur = (int32_t *)malloc(cap * sizeof(int32_t));
  int32_t *tmp = (int32_t *)malloc(cap * sizeof(int32_t));
  int32_t *where = NULL; /* column -> position inside the current vector-row */
  if (vec_val) {
    where = (int32_t *)malloc((size_t)(K > 0 ? K : 1) * sizeof(int32_t));
  }
  for (int32_t i = 0; i < m_vec; ++i) {
    int64_t ncur = 0;
    for (int32_t j = 0; j < V; ++j) {
      int64_t r = (int64_t)i * V + j;
      if (r >= M) continue; /* sparse_matrix_format.py:109 */
      int64_t b = row_ptr[r], e = row_ptr[r + 1];
      int64_t need = ncur + (e - b);
      if (need > cap) {
        while (cap < need) cap *= 2;
        cur = (int32_t *)realloc(cur, cap * sizeof(int32_t));
        tmp = (int32_t *)realloc(tmp, cap * sizeof(int32_t));
      }
      /* vec_colInd + colInd_list_array[r] */
      memcpy(tmp, cur, ncur * sizeof(int32_t));
      memcpy(tmp + ncur, col_ind + b, (e - b) * sizeof(int32_t));
      if (order == 0) {
        ncur = oracle_pyset_order(tmp, need, cur);
      } else {
        qsort(tmp, need, sizeof(int32_t), cmp_i32);
        ncur = 0;
        for (int64_t t = 0; t < need; ++t)
          if (t == 0 || tmp[t] != tmp[t - 1]) cur[ncur++] = tmp[t];
      }
    }
    if (vec_col) memcpy(vec_col + nvec, cur, ncur * sizeof(int32_t));
    if (vec_val) {
      memset(vec_val + nvec * V, 0, (size_t)ncur * V * sizeof(uint16_t));
      for (int64_t p = 0; p < ncur; ++p) where[cur[p]] = (int32_t)p;
      for (int32_t j = 0; j < V; ++j) {
        int64_t r = (int64_t)i * V + j;
        if (r >= M) continue;
        for (int64_t t = row_ptr[r]; t < row_ptr[r + 1]; ++t)
          vec_val[(nvec + where[col_ind[t]]) * V + j] = csr_val[t];
      }
    }
    nvec += ncur;
    vec_row_ptr[i + 1] = (int32_t)nvec;
  }
  free(cur);
  free(tmp);
  free(where);
  return nvec;
}

/* ------------------------------------------------------------------ SpMM */

/*
 * C[(i*V+v)*N + l] += float(values[j*V+v]) * float(B[col_j*N + l]), j ascending,
 * fp32 accumulate, C zero-initialised (sspmm_test.cpp:75-95).  threads > 1
 * splits vector-rows over OpenMP threads (same per-element order, so the result
 * is identical).
 */
void oracle_spmm_f32(int32_t m_vec, int32_t V, int32_t N, int32_t K, const int32_t *row_offsets,
                     const int32_t *col_idx, const uint16_t *values, const uint16_t *B, float *C,
                     int32_t threads) {
  (void)K;
  if (threads < 1) threads = 1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
  for (int32_t i = 0; i < m_vec; ++i) {
    float *brow = (float *)malloc((size_t)N * sizeof(float));
    for (int32_t v = 0; v < V; ++v)
      for (int32_t l = 0; l < N; ++l) C[((int64_t)i * V + v) * N + l] = 0.0f;
    for (int32_t j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
      int32_t col = col_idx[j];
      for (int32_t l = 0; l < N; ++l) brow[l] = h2f(B[(int64_t)col * N + l]);
      for (int32_t v = 0; v < V; ++v) {
        float a = h2f(values[(int64_t)j * V + v]);
        float *c = C + ((int64_t)i * V + v) * N;
        for (int32_t l = 0; l < N; ++l) c[l] += a * brow[l];
      }
    }
    free(brow);
  }
}

/* fp16 output: the fp32 result rounded to nearest even. */
void oracle_spmm_f16(int32_t m_vec, int32_t V, int32_t N, int32_t K, const int32_t *row_offsets,
                     const int32_t *col_idx, const uint16_t *values, const uint16_t *B, uint16_t *C,
                     int32_t threads) {
  int64_t total = (int64_t)m_vec * V * N;
  float *tmp = (float *)malloc((size_t)(total > 0 ? total : 1) * sizeof(float));
  oracle_spmm_f32(m_vec, V, N, K, row_offsets, col_idx, values, B, tmp, threads);
  for (int64_t t = 0; t < total; ++t) C[t] = f2h_rn(tmp[t]);
  free(tmp);
}

/* ---------------------------------------------------------- row swizzle */

typedef struct {
  int32_t len, idx;
} lenidx;

static int cmp_lenidx_desc(const void *a, const void *b) {
  const lenidx *x = (const lenidx *)a, *y = (const lenidx *)b;
  if (x->len != y->len) return (x->len < y->len) - (x->len > y->len);
  return (x->idx > y->idx) - (x->idx < y->idx);
}

void oracle_sorted_row_swizzle(int32_t rows, const int32_t *row_offsets, int32_t *row_indices) {
  lenidx *t = (lenidx *)malloc((size_t)(rows > 0 ? rows : 1) * sizeof(lenidx));
  for (int32_t i = 0; i < rows; ++i) {
    t[i].len = row_offsets[i + 1] - row_offsets[i];
    t[i].idx = i;
  }
  qsort(t, rows, sizeof(lenidx), cmp_lenidx_desc);
  for (int32_t i = 0; i < rows; ++i) row_indices[i] = t[i].idx;
  free(t);
}

/* -------------------------------------------------------- row reordering */

static uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x85ebca6bu;
  x ^= x >> 13;
  x *= 0xc2b2ae35u;
  x ^= x >> 16;
  return x;
}

typedef struct {
  uint64_t key;
  int32_t idx;
} keyidx;

static int cmp_keyidx(const void *a, const void *b) {
  const keyidx *x = (const keyidx *)a, *y = (const keyidx *)b;
  if (x->key != y->key) return (x->key > y->key) - (x->key < y->key);
  return (x->idx > y->idx) - (x->idx < y->idx);
}

/* keys[i] = min over the row's columns of mix32(c ^ seed1), << 32, | the same with seed2;
 * perm = argsort of the keys, ties by ascending row.  keys may be NULL. */
void oracle_minhash_order(int32_t M, const int32_t *row_ptr, const int32_t *col_ind, int32_t *perm, uint64_t *keys) {
  keyidx *t = (keyidx *)malloc((size_t)(M > 0 ? M : 1) * sizeof(keyidx));
  for (int32_t i = 0; i < M; ++i) {
    uint32_t h1 = 0xffffffffu, h2 = 0xffffffffu;
    for (int32_t e = row_ptr[i]; e < row_ptr[i + 1]; ++e) {
      const uint32_t c = (uint32_t)col_ind[e];
      const uint32_t a = mix32(c ^ 0x9e3779b9u), b = mix32(c ^ 0x7f4a7c15u);
      if (a < h1) h1 = a;
      if (b < h2) h2 = b;
    }
    t[i].key = ((uint64_t)h1 << 32) | h2;
    t[i].idx = i;
    if (keys) keys[i] = t[i].key;
  }
  qsort(t, M, sizeof(keyidx), cmp_keyidx);
  for (int32_t i = 0; i < M; ++i) perm[i] = t[i].idx;
  free(t);
}

/* out row i = source row perm[i]; val / out_val may be NULL. */
void oracle_permute_csr(int32_t M, const int32_t *perm, const int32_t *row_ptr, const int32_t *col_ind,
                        const uint16_t *val, int32_t *out_row_ptr, int32_t *out_col, uint16_t *out_val) {
  out_row_ptr[0] = 0;
  for (int32_t i = 0; i < M; ++i) {
    const int32_t s0 = row_ptr[perm[i]], n = row_ptr[perm[i] + 1] - s0, d0 = out_row_ptr[i];
    memcpy(out_col + d0, col_ind + s0, (size_t)n * sizeof(int32_t));
    if (val) memcpy(out_val + d0, val + s0, (size_t)n * sizeof(uint16_t));
    out_row_ptr[i + 1] = d0 + n;
  }
}

/* ------------------------------------------------- sparse attention steps */

/* lhs[M x F], rhs[n_rhs x F] fp16 row-major; out[nvec*V] fp16. */
void oracle_sddmm_f16(int32_t m_vec, int32_t V, int32_t F, const int32_t *row_offsets, const int32_t *col_idx,
                      const uint16_t *lhs, const uint16_t *rhs, uint16_t *out) {
  for (int32_t i = 0; i < m_vec; ++i)
    for (int32_t j = row_offsets[i]; j < row_offsets[i + 1]; ++j)
      for (int32_t v = 0; v < V; ++v) {
        const uint16_t *a = lhs + ((int64_t)i * V + v) * F, *b = rhs + (int64_t)col_idx[j] * F;
        float acc = 0.f;
        for (int32_t f = 0; f < F; ++f) acc += h2f(a[f]) * h2f(b[f]);
        out[(int64_t)j * V + v] = f2h_rn(acc);
      }
}

/* values[nvec*V] fp16 -> out[nvec*V] fp16; a vector-row without vectors writes nothing. */
void oracle_softmax_f16(int32_t m_vec, int32_t V, const int32_t *row_offsets, const uint16_t *values, float scaler,
                        uint16_t *out) {
  for (int32_t i = 0; i < m_vec; ++i)
    for (int32_t v = 0; v < V; ++v) {
      const int32_t b = row_offsets[i], e = row_offsets[i + 1];
      if (b == e) continue;
      float mx = -INFINITY, sum = 0.f;
      for (int32_t j = b; j < e; ++j) {
        const float x = h2f(values[(int64_t)j * V + v]) * scaler;
        mx = x > mx ? x : mx;
      }
      for (int32_t j = b; j < e; ++j) sum += expf(h2f(values[(int64_t)j * V + v]) * scaler - mx);
      for (int32_t j = b; j < e; ++j)
        out[(int64_t)j * V + v] = f2h_rn(expf(h2f(values[(int64_t)j * V + v]) * scaler - mx) / sum);
    }
}

/*
 * CPU restatement of the reference's six sparse-FlashAttention kernels.
 * TEST INFRASTRUCTURE ONLY: nothing in the shipped library links or loads this file.
 * It is used by tests/, by the smoke check and by the cpu_baseline leg of the benchmark.
 *
 * Every reference kernel is one thread block per query row running the same loop
 * (Sparse_FlashAttention_CSR/sp_flatt_csr_kernel.cu:14-220); the six kernels differ only
 * in where a row's list of live columns comes from.  This file restates that loop once
 * (row_attend) in double precision and restates the six column rules around it.
 *
 * Deliberate departures from the reference source (its defects, not its algorithm):
 *   - the last chunk of a row is sized "what is left" instead of "tot % chunk", so a row
 *     whose length is an exact multiple of the chunk is not cut short
 *     (sp_flatt_csr_kernel.cu:101,107-109);
 *   - dilated column t of a row is low + t*s for the row-wide t, so later chunks do not
 *     re-read wrong columns (sp_flatt_local_1d_dilated_kernel.cu:102,111);
 *   - COO rows are located by bucketing instead of two linear scans
 *     (sp_flatt_coo_kernel.cu:47-79), which also makes unsorted input well defined;
 *   - a row of the global mask that ends up with no live column is left untouched
 *     instead of dividing by zero (sp_flatt_global_no_local_kernel.cu:83-85).
 *
 * How it is pinned: tests compare it with the float64 numpy dense formulation, with the
 * committed golden vectors written by torch's scaled_dot_product_attention, and with the
 * closed forms (window 0 => out == v; V == 1 => out == 1).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define SPFA_ORACLE_OK 0
#define SPFA_ORACLE_ERR_EMB 5
#define SPFA_ORACLE_ERR_LOCAL 6
#define SPFA_ORACLE_ERR_DIL 7
#define SPFA_ORACLE_ERR_BLOCK_DIV 8
#define SPFA_ORACLE_ERR_BLOCK_DIL 9
#define SPFA_ORACLE_ERR_GLOBS 10

typedef struct {
  int64_t n, d;
  const double *q, *k, *v;
  double *m, *l, *out;
  int chunk;
} ctx_t;

/* column t of the current row */
typedef int64_t (*col_fn)(const void *row_state, int64_t t);

/*
 * One query row.  Mirrors sp_flatt_csr_kernel.cu: load Q row, the row of O already in
 * memory and its m, l (:79-92); per chunk: scores q.k/sqrt(d) (:130-138), chunk max
 * (:142-152), exponentials (:156-158), chunk sum and the merged statistics (:162-179),
 * P.V and the renormalised O (:184-194), carry (:198-201); finally write m, l, O back
 * (:208-218).  O is kept normalised after every chunk, as in the reference.
 */
static void row_attend(const ctx_t *c, int64_t row, int64_t tot, col_fn col, const void *rs,
                       double *w, double *acc) {
  const int64_t d = c->d;
  const double *qi = c->q + row * d;
  double *oi = c->out + row * d;
  double m_i = c->m[row];
  double l_i = c->l[row];
  const double inv = 1.0 / sqrt((double)d);
  int64_t done = 0;
  while (done < tot) {
    int64_t cnt = tot - done;
    if (cnt > c->chunk) cnt = c->chunk;
    double m_ij = -INFINITY;
    for (int64_t t = 0; t < cnt; t++) {
      const double *kj = c->k + col(rs, done + t) * d;
      double a = 0.0;
      for (int64_t e = 0; e < d; e++) a += qi[e] * kj[e];
      w[t] = a * inv;
      if (w[t] > m_ij) m_ij = w[t];
    }
    double l_ij = 0.0;
    for (int64_t t = 0; t < cnt; t++) {
      w[t] = exp(w[t] - m_ij);
      l_ij += w[t];
    }
    double m_new = m_i > m_ij ? m_i : m_ij;
    /* a state with l == 0 carries no weight whatever its m and O hold */
    double wa = (l_i != 0.0) ? l_i * exp(m_i - m_new) : 0.0;
    double eb = exp(m_ij - m_new);
    double l_new = wa + l_ij * eb;
    for (int64_t e = 0; e < d; e++) acc[e] = 0.0;
    for (int64_t t = 0; t < cnt; t++) {
      const double *vj = c->v + col(rs, done + t) * d;
      for (int64_t e = 0; e < d; e++) acc[e] += w[t] * vj[e];
    }
    for (int64_t e = 0; e < d; e++) {
      double prev = (wa != 0.0) ? wa * oi[e] : 0.0;
      oi[e] = (1.0 / l_new) * (prev + acc[e] * eb);
    }
    m_i = m_new;
    l_i = l_new;
    done += cnt;
  }
  c->m[row] = m_i;
  c->l[row] = l_i;
}

static void nan_fill(const ctx_t *c, int64_t row) {
  for (int64_t e = 0; e < c->d; e++) c->out[row * c->d + e] = NAN;
}

/* ------------------------------------------------------------------ CSR */
typedef struct { const int64_t *cols; } list_state;
static int64_t col_list(const void *rs, int64_t t) { return ((const list_state *)rs)->cols[t]; }

/* sp_flatt_csr_kernel.cu:29-33 (row bounds), :45-54 (empty row), :117 (column) */
int spfa_oracle_csr(int64_t n, int64_t d, const double *q, const double *k, const double *v,
                    const int64_t *row_off, const int64_t *col_ind, double *m, double *l,
                    double *out, int use_nan, int chunk) {
  if (chunk < 1) return SPFA_ORACLE_ERR_EMB;
  ctx_t c = {n, d, q, k, v, m, l, out, chunk};
#pragma omp parallel
  {
    double *w = (double *)malloc(sizeof(double) * (size_t)chunk);
    double *acc = (double *)malloc(sizeof(double) * (size_t)d);
#pragma omp for schedule(dynamic, 16)
    for (int64_t i = 0; i < n; i++) {
      int64_t low = row_off[i], up = row_off[i + 1];
      int64_t tot = up - low;
      if (tot == 0) {
        if (use_nan) nan_fill(&c, i);
        continue;
      }
      list_state rs = {col_ind + low};
      row_attend(&c, i, tot, col_list, &rs, w, acc);
    }
    free(w);
    free(acc);
  }
  return SPFA_ORACLE_OK;
}

/* ------------------------------------------------------------------ COO */
/* live(i) = { col[p] : row[p] == i } - the row range of sp_flatt_coo_kernel.cu:47-84 */
int spfa_oracle_coo(int64_t n, int64_t d, const double *q, const double *k, const double *v,
                    const int64_t *row_ind, const int64_t *col_ind, int64_t nnz, double *m,
                    double *l, double *out, int use_nan, int chunk) {
  int64_t *off = (int64_t *)calloc((size_t)n + 1, sizeof(int64_t));
  int64_t *cur = (int64_t *)malloc(sizeof(int64_t) * ((size_t)n + 1));
  int64_t *cols = (int64_t *)malloc(sizeof(int64_t) * (size_t)(nnz > 0 ? nnz : 1));
  for (int64_t p = 0; p < nnz; p++) off[row_ind[p] + 1]++;
  for (int64_t i = 0; i < n; i++) off[i + 1] += off[i];
  memcpy(cur, off, sizeof(int64_t) * ((size_t)n + 1));
  for (int64_t p = 0; p < nnz; p++) cols[cur[row_ind[p]]++] = col_ind[p];
  int rc = spfa_oracle_csr(n, d, q, k, v, off, cols, m, l, out, use_nan, chunk);
  free(off);
  free(cur);
  free(cols);
  return rc;
}

/* ------------------------------------------------------------------ strided bands */
typedef struct { int64_t low, stride; } stride_state;
static int64_t col_stride(const void *rs, int64_t t) {
  const stride_state *s = (const stride_state *)rs;
  return s->low + t * s->stride;
}

/* sp_flatt_local_kernel.cu:24-28 (bounds), :101 (column), :252-254 (check) */
int spfa_oracle_local(int64_t n, int64_t d, const double *q, const double *k, const double *v,
                      double *m, double *l, double *out, int64_t w, int chunk) {
  if (chunk < 1) return SPFA_ORACLE_ERR_EMB;
  if (w < 0 || w > n - 1) return SPFA_ORACLE_ERR_LOCAL;
  ctx_t c = {n, d, q, k, v, m, l, out, chunk};
#pragma omp parallel
  {
    double *wb = (double *)malloc(sizeof(double) * (size_t)chunk);
    double *acc = (double *)malloc(sizeof(double) * (size_t)d);
#pragma omp for schedule(dynamic, 16)
    for (int64_t i = 0; i < n; i++) {
      int64_t low = i - w > 0 ? i - w : 0;
      int64_t up = i + w + 1 < n ? i + w + 1 : n;
      stride_state rs = {low, 1};
      row_attend(&c, i, up - low, col_stride, &rs, wb, acc);
    }
    free(wb);
    free(acc);
  }
  return SPFA_ORACLE_OK;
}

/* sp_flatt_local_1d_dilated_kernel.cu:25-29 (bounds), :102 (column), :254-261 (checks) */
int spfa_oracle_local_1d_dilated(int64_t n, int64_t d, const double *q, const double *k,
                                 const double *v, double *m, double *l, double *out, int64_t w,
                                 int64_t dil, int chunk) {
  if (chunk < 1) return SPFA_ORACLE_ERR_EMB;
  if (w < 0 || w > n - 1) return SPFA_ORACLE_ERR_LOCAL;
  if (dil < 0) return SPFA_ORACLE_ERR_DIL;
  const int64_t s = dil + 1;
  ctx_t c = {n, d, q, k, v, m, l, out, chunk};
#pragma omp parallel
  {
    double *wb = (double *)malloc(sizeof(double) * (size_t)chunk);
    double *acc = (double *)malloc(sizeof(double) * (size_t)d);
#pragma omp for schedule(dynamic, 16)
    for (int64_t i = 0; i < n; i++) {
      int64_t low = i - w * s > i % s ? i - w * s : i % s;
      int64_t up = i + w * s < n - 1 ? i + w * s : n - 1;
      int64_t tot = (up - low) / s + 1;
      stride_state rs = {low, s};
      row_attend(&c, i, tot, col_stride, &rs, wb, acc);
    }
    free(wb);
    free(acc);
  }
  return SPFA_ORACLE_OK;
}

/* sp_flatt_local_2d_dilated_kernel.cu:26-39 (block, live rows), :51-60 (dead rows),
 * :123 (column), :274-286 (checks) */
int spfa_oracle_local_2d_dilated(int64_t n, int64_t d, const double *q, const double *k,
                                 const double *v, double *m, double *l, double *out,
                                 int64_t block, int64_t dil, int use_nan, int chunk) {
  if (chunk < 1) return SPFA_ORACLE_ERR_EMB;
  if (block <= 0 || n % block != 0) return SPFA_ORACLE_ERR_BLOCK_DIV;
  if (dil < 0) return SPFA_ORACLE_ERR_DIL;
  if (block / (dil + 1) < 1) return SPFA_ORACLE_ERR_BLOCK_DIL;
  const int64_t s = dil + 1;
  ctx_t c = {n, d, q, k, v, m, l, out, chunk};
#pragma omp parallel
  {
    double *wb = (double *)malloc(sizeof(double) * (size_t)chunk);
    double *acc = (double *)malloc(sizeof(double) * (size_t)d);
#pragma omp for schedule(dynamic, 16)
    for (int64_t i = 0; i < n; i++) {
      int64_t low = (i / block) * block;
      int64_t tot = 0;
      if ((i - low) % s == 0) {
        tot = (block - 1) / s + 1;
        if (tot > block) tot = block;
      }
      if (tot == 0) {
        if (use_nan) nan_fill(&c, i);
        continue;
      }
      stride_state rs = {low, s};
      row_attend(&c, i, tot, col_stride, &rs, wb, acc);
    }
    free(wb);
    free(acc);
  }
  return SPFA_ORACLE_OK;
}

/* ------------------------------------------------------------------ global minus local */
typedef struct { int64_t low, win; } hole_state;
static int64_t col_hole(const void *rs, int64_t t) {
  const hole_state *h = (const hole_state *)rs;
  return t < h->low ? t : t + h->win;
}

/* sp_flatt_global_no_local_kernel.cu:38-39 (window), :47-64 (row class and count),
 * :134-162 (column map), :325-334 (checks) */
int spfa_oracle_global_no_local(int64_t n, int64_t d, const double *q, const double *k,
                                const double *v, double *m, double *l, double *out,
                                const int32_t *globs, int64_t n_globs, int64_t w, int chunk) {
  if (chunk < 1) return SPFA_ORACLE_ERR_EMB;
  if (n_globs == 0 || n_globs > n) return SPFA_ORACLE_ERR_GLOBS;
  if (w < 0 || w > n - 1) return SPFA_ORACLE_ERR_LOCAL;
  ctx_t c = {n, d, q, k, v, m, l, out, chunk};
#pragma omp parallel
  {
    double *wb = (double *)malloc(sizeof(double) * (size_t)chunk);
    double *acc = (double *)malloc(sizeof(double) * (size_t)d);
    int64_t *lst = (int64_t *)malloc(sizeof(int64_t) * (size_t)n_globs);
#pragma omp for schedule(dynamic, 16)
    for (int64_t i = 0; i < n; i++) {
      int64_t low = i - w > 0 ? i - w : 0;
      int64_t up = i + w + 1 < n ? i + w + 1 : n;
      int is_global = 0;
      int64_t cnt = 0;
      for (int64_t g = 0; g < n_globs; g++) {
        int64_t t = globs[g];
        if (t == i) {
          is_global = 1;
          break;
        } else if (t < low || t > up - 1) {
          lst[cnt++] = t;
        }
      }
      if (is_global) {
        hole_state rs = {low, up - low};
        int64_t tot = n - (up - low);
        if (tot > 0) row_attend(&c, i, tot, col_hole, &rs, wb, acc);
      } else if (cnt > 0) {
        list_state rs = {lst};
        row_attend(&c, i, cnt, col_list, &rs, wb, acc);
      }
    }
    free(wb);
    free(acc);
    free(lst);
  }
  return SPFA_ORACLE_OK;
}

/* C restatement of the reference's f32 log-space CPU kernel on a flattened SPN.
 *
 * TEST INFRASTRUCTURE ONLY: used by tests/ and bench.py's cpu_baseline leg as a checker,
 * never linked into or called from the product library.
 *
 * Follows, per node kind:
 *   product  balanced binary tree of adds, pivot ceil(k/2), left first
 *            (mlir/lib/Conversion/HiSPNtoLoSPN/NodePatterns.cpp:17-40; log-space mul = addf,
 *             mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:182-197)
 *   sum      child + (float)log(w) per child, then the same balanced tree of log-adds
 *            a + log1p(exp(b - a)), a = x OGT y ? x : y
 *            (HiSPNtoLoSPN/NodePatterns.cpp:49-88, LoSPNtoCPU/NodePatterns.cpp:216-240)
 *   gaussian coef + ((x-mean)*(x-mean))*den, coef = -ln(sd) - 0.5 ln(2 pi), den = -1/(2 sd^2),
 *            constants computed in double and rounded once (LoSPNtoCPU/NodePatterns.cpp:306-374)
 *   table    T[i] = (float)log(p_i), index = fptoui(x) (LoSPNtoCPU/NodePatterns.cpp:376-529);
 *            an index outside the table gives -inf (the reference's GPU lowering,
 *            mlir/lib/Conversion/LoSPNtoGPU/GPUNodePatterns.cpp:385-395; its CPU lowering does
 *            not check)
 *   marginal NaN input -> leaf value 0 (select after the computation)
 * Parity status: pinned through tests/test_oracle_pins.py (known answers of
 * execute/src/main.cpp:32-52, the NIPS5 / nltcs / plants golden outputs, FileCheck constants).
 */
#include <math.h>
#include <omp.h>
#include <stdlib.h>
#include <stddef.h>

enum { K_PRODUCT = 0, K_SUM = 1, K_HISTOGRAM = 2, K_GAUSSIAN = 3, K_CATEGORICAL = 4 };

typedef struct {
  int num_nodes;          /* topological order, root last */
  int num_features;
  const int* kind;        /* [num_nodes] */
  const int* column;      /* [num_nodes] input column of a leaf */
  const double* mean;     /* [num_nodes] */
  const double* stddev;   /* [num_nodes] */
  const int* table_off;   /* [num_nodes] offset into tables (linear probabilities) */
  const int* table_len;   /* [num_nodes] */
  const double* tables;
  const int* child_off;   /* [num_nodes] offset into children / weights */
  const int* child_cnt;   /* [num_nodes] */
  const int* children;    /* node indices */
  const double* weights;  /* linear weights, aligned with children */
} spn_flat;

static float logadd(float x, float y) {
  const int gt = x > y;
  const float a = gt ? x : y;
  const float b = gt ? y : x;
  return a + log1pf(expf(b - a));
}

static float tree(const float* t, int lo, int hi, int is_sum) {
  const int k = hi - lo;
  if (k == 1) return t[lo];
  if (k == 2) return is_sum ? logadd(t[lo], t[lo + 1]) : t[lo] + t[lo + 1];
  const int pivot = lo + (k + 1) / 2;
  const float l = tree(t, lo, pivot, is_sum), r = tree(t, pivot, hi, is_sum);
  return is_sum ? logadd(l, r) : l + r;
}

/* Threads the sample loop runs on, and a way to time a single one (bench.py's cpu_baseline). */
int spn_oracle_threads(void) { return omp_get_max_threads(); }
void spn_oracle_set_threads(int n) { omp_set_num_threads(n); }

/* in: [n, num_features] as double (integers exactly representable); out: [n] float. */
int spn_oracle_f32(const spn_flat* s, const double* in, size_t n, int marginal, float* out) {
  int max_k = 1;
  for (int i = 0; i < s->num_nodes; ++i)
    if (s->child_cnt[i] > max_k) max_k = s->child_cnt[i];
  /* constants, rounded once from double */
  float* ftab = NULL;
  int total_tab = 0;
  for (int i = 0; i < s->num_nodes; ++i)
    if (s->table_off[i] + s->table_len[i] > total_tab) total_tab = s->table_off[i] + s->table_len[i];
  ftab = (float*)malloc(sizeof(float) * (size_t)(total_tab > 0 ? total_tab : 1));
  for (int i = 0; i < total_tab; ++i) ftab[i] = (float)log(s->tables[i]);
  int failed = 0;
#pragma omp parallel
  {
    float* val = (float*)malloc(sizeof(float) * (size_t)s->num_nodes);
    float* tmp = (float*)malloc(sizeof(float) * (size_t)max_k);
    if (!val || !tmp) {
#pragma omp atomic write
      failed = 1;
    } else {
#pragma omp for schedule(static)
      for (long r = 0; r < (long)n; ++r) {
        const double* x = in + (size_t)r * (size_t)s->num_features;
        for (int i = 0; i < s->num_nodes; ++i) {
          float v;
          switch (s->kind[i]) {
            case K_GAUSSIAN: {
              const float xf = (float)x[s->column[i]];
              const float coef = (float)(-log(s->stddev[i]) + -0.5 * log(2.0 * M_PI));
              const float den = (float)(-(1.0 / (2.0 * s->stddev[i] * s->stddev[i])));
              const float d = xf - (float)s->mean[i];
              v = coef + (d * d) * den;
              if (marginal && xf != xf) v = 0.0f;
              break;
            }
            case K_CATEGORICAL:
            case K_HISTOGRAM: {
              const double xv = x[s->column[i]];
              if (xv != xv) {
                v = marginal ? 0.0f : -INFINITY;
              } else if (xv > -1.0 && xv < (double)s->table_len[i]) {
                v = ftab[s->table_off[i] + (int)xv];
              } else {
                v = -INFINITY;
              }
              break;
            }
            case K_PRODUCT: {
              const int k = s->child_cnt[i], off = s->child_off[i];
              for (int j = 0; j < k; ++j) tmp[j] = val[s->children[off + j]];
              v = tree(tmp, 0, k, 0);
              break;
            }
            default: { /* K_SUM */
              const int k = s->child_cnt[i], off = s->child_off[i];
              for (int j = 0; j < k; ++j) tmp[j] = val[s->children[off + j]] + (float)log(s->weights[off + j]);
              v = tree(tmp, 0, k, 1);
              break;
            }
          }
          val[i] = v;
        }
        out[r] = val[s->num_nodes - 1];
      }
    }
    free(val);
    free(tmp);
  }
  free(ftab);
  return failed;
}

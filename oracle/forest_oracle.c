/*
 * CPU oracle for decision-forest inference.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C restatement of the scalar reference semantics of
 * asprasad/treebeard.  It is the checker that the GPU library is compared
 * against; it is never linked into, called from or shipped with the product
 * library.  Only tests/, the smoke check and the CPU-baseline leg of the
 * benchmark may load it.
 *
 * Reference functions followed (paths relative to the reference checkout):
 *   src/include/DecisionForest.h:347-364  DecisionTree::PredictTree       (double walk)
 *   src/include/DecisionForest.h:366-379  DecisionTree::PredictTree_Float (f32 walk)
 *   src/include/DecisionForest.h:442-444  sigmoid
 *   src/include/DecisionForest.h:446-468  argmax (std::max_element: first maximum)
 *   src/include/DecisionForest.h:470-502  DecisionForest::Predict
 *   src/include/DecisionForest.h:504-536  DecisionForest::Predict_Float
 *   src/mlir/LowerReduceOps.cpp:148-187   generated-code argmax (tie -> larger id)
 *   src/mlir/ReorderTiledTreesByDepth.cpp:387-398  batch split over cores
 *
 * Pinning (what each function is checked against in tests/):
 *   oracle_leaf_ids / oracle_predict      - the reference's own header compiled
 *       into oracle/_ref (DecisionForest::Predict / Predict_Float), the
 *       XGBoost golden CSVs the reference ships, brute-force python walks.
 *   sigmoid                               - scipy.special.expit, golden CSVs
 *   argmax                                - numpy argmax + explicit tie cases
 *   softmax probabilities                 - PARITY UNPINNED in the reference
 *       (it never computes them); closed form scipy.special.softmax only.
 *
 * Forest layout (all arrays caller-owned, node indices local to each tree):
 *   tree_offsets[num_trees+1]  first node of each tree in the flat arrays
 *   threshold[n]  double; already rounded to f32 by the loader when the
 *                 threshold type is f32 (xgboostparser.h:205 get<float>())
 *   feature[n]    int32; ignored on leaves
 *   left[n], right[n]  int32 local child index, -1 on leaves
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct {
  int32_t num_trees;
  int32_t num_features;
  int32_t num_classes;   /* 0 = regression / binary */
  int32_t transform;     /* 0 identity, 1 sigmoid, 2 softmax(argmax) */
  int32_t predicate;     /* 0: x<thr -> left, 1: x>=thr, 2: x>thr, 3: x<=thr */
  double initial_value;
  const int64_t *tree_offsets;
  const double *threshold;
  const int32_t *feature;
  const int32_t *left;
  const int32_t *right;
  const int32_t *class_id; /* per tree */
} oracle_forest_t;

static inline int goes_left_f32(int predicate, float x, float thr) {
  switch (predicate) {
  case 0: return x < thr;
  case 1: return x >= thr;
  case 2: return x > thr;
  default: return x <= thr;
  }
}

/* DecisionForest.h:366-379.  Returns the local node id of the leaf reached. */
static inline int32_t walk_tree_f32(const oracle_forest_t *f, int32_t t,
                                    const float *row, int32_t *steps) {
  const int64_t base = f->tree_offsets[t];
  int32_t n = 0, s = 0;
  while (!(f->left[base + n] == -1 && f->right[base + n] == -1)) {
    float thr = (float)f->threshold[base + n];
    if (goes_left_f32(f->predicate, row[f->feature[base + n]], thr))
      n = f->left[base + n];
    else
      n = f->right[base + n];
    ++s;
  }
  if (steps) *steps = s;
  return n;
}

/* DecisionForest.h:347-364, the double-precision twin. */
static inline int32_t walk_tree_f64(const oracle_forest_t *f, int32_t t,
                                    const double *row) {
  const int64_t base = f->tree_offsets[t];
  int32_t n = 0;
  while (!(f->left[base + n] == -1 && f->right[base + n] == -1)) {
    double thr = f->threshold[base + n], x = row[f->feature[base + n]];
    int l;
    switch (f->predicate) {
    case 0: l = x < thr; break;
    case 1: l = x >= thr; break;
    case 2: l = x > thr; break;
    default: l = x <= thr; break;
    }
    n = l ? f->left[base + n] : f->right[base + n];
  }
  return n;
}

/* Leaf node id for every (row, tree); optional path length per (row, tree). */
void oracle_leaf_ids(const oracle_forest_t *f, const float *x, int64_t rows,
                     int32_t *leaf_ids, int32_t *path_len, int32_t threads) {
  const int32_t T = f->num_trees, F = f->num_features;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    for (int32_t t = 0; t < T; ++t) {
      int32_t s;
      leaf_ids[r * T + t] = walk_tree_f32(f, t, x + r * F, &s);
      if (path_len) path_len[r * T + t] = s;
    }
  }
}

/* Total visited internal nodes over all (row, tree) pairs. */
int64_t oracle_total_steps(const oracle_forest_t *f, const float *x,
                           int64_t rows, int32_t threads) {
  const int32_t T = f->num_trees, F = f->num_features;
  int64_t total = 0;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) reduction(+ : total) schedule(static)
  for (int64_t r = 0; r < rows; ++r)
    for (int32_t t = 0; t < T; ++t) {
      int32_t s;
      (void)walk_tree_f32(f, t, x + r * F, &s);
      total += s;
    }
  return total;
}

static inline double sigmoid_f64(double v) { return 1.0 / (1.0 + exp(-v)); }

/*
 * DecisionForest::Predict_Float (DecisionForest.h:504-536).
 *   regression / binary: leaf values are narrowed to float, accumulated in
 *     tree order into a DOUBLE that starts at the initial value
 *     (std::accumulate with a double init), transformed, narrowed to float.
 *   multiclass: per class, double accumulate (starting at the initial value)
 *     of that class's leaves in tree order; result is the index of the first
 *     maximum of the sums *after each was narrowed to float* (the vector is
 *     std::vector<float>).
 * out_pred   f32[rows]            prediction (class id as float for multiclass)
 * out_sums   f64[rows][max(1,C)]  raw margin(s) before the transform, optional
 */
void oracle_predict_f32(const oracle_forest_t *f, const float *x, int64_t rows,
                        float *out_pred, double *out_sums, int32_t threads) {
  const int32_t T = f->num_trees, F = f->num_features, C = f->num_classes;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float *row = x + r * F;
    if (C == 0) {
      double acc = f->initial_value;
      for (int32_t t = 0; t < T; ++t) {
        int32_t n = walk_tree_f32(f, t, row, NULL);
        acc += (double)(float)f->threshold[f->tree_offsets[t] + n];
      }
      if (out_sums) out_sums[r] = acc;
      if (f->transform == 1)
        out_pred[r] = (float)sigmoid_f64(acc);
      else
        out_pred[r] = (float)acc;
    } else {
      double sums[256];
      int seen[256];
      for (int32_t c = 0; c < C; ++c) { sums[c] = f->initial_value; seen[c] = 0; }
      for (int32_t t = 0; t < T; ++t) {
        int32_t n = walk_tree_f32(f, t, row, NULL);
        int32_t c = f->class_id[t];
        sums[c] += (double)(float)f->threshold[f->tree_offsets[t] + n];
        seen[c] = 1;
      }
      /* classes with no trees keep probability 0 (vector initialised to 0) */
      int32_t best = 0;
      float bestv = 0.f;
      for (int32_t c = 0; c < C; ++c) {
        float v = seen[c] ? (float)sums[c] : 0.f;
        if (out_sums) out_sums[r * C + c] = seen[c] ? sums[c] : 0.0;
        if (c == 0 || v > bestv) { best = c; bestv = v; }
      }
      out_pred[r] = (float)best;
    }
  }
}

/* DecisionForest::Predict (DecisionForest.h:470-502): everything in double. */
void oracle_predict_f64(const oracle_forest_t *f, const double *x, int64_t rows,
                        double *out_pred) {
  const int32_t T = f->num_trees, F = f->num_features, C = f->num_classes;
  for (int64_t r = 0; r < rows; ++r) {
    const double *row = x + r * F;
    if (C == 0) {
      double acc = f->initial_value;
      for (int32_t t = 0; t < T; ++t)
        acc += f->threshold[f->tree_offsets[t] + walk_tree_f64(f, t, row)];
      out_pred[r] = f->transform == 1 ? sigmoid_f64(acc) : acc;
    } else {
      double sums[256];
      int seen[256];
      for (int32_t c = 0; c < C; ++c) { sums[c] = f->initial_value; seen[c] = 0; }
      for (int32_t t = 0; t < T; ++t) {
        int32_t c = f->class_id[t];
        sums[c] += f->threshold[f->tree_offsets[t] + walk_tree_f64(f, t, row)];
        seen[c] = 1;
      }
      int32_t best = 0;
      double bestv = 0;
      for (int32_t c = 0; c < C; ++c) {
        double v = seen[c] ? sums[c] : 0.0;
        if (c == 0 || v > bestv) { best = c; bestv = v; }
      }
      out_pred[r] = (double)best;
    }
  }
}

/*
 * Generated-code argmax (LowerReduceOps.cpp:148-187, :511-516): running
 * maximum starts at -inf / index 0 and is replaced unless `max > cur`
 * (ordered greater-than), so on exact ties the LARGER class id wins.
 * sums: f32[rows][C].
 */
void oracle_argmax_generated(const float *sums, int64_t rows, int32_t C,
                             int8_t *out) {
  for (int64_t r = 0; r < rows; ++r) {
    float mx = -INFINITY;
    int32_t idx = 0;
    for (int32_t c = 0; c < C; ++c) {
      float cur = sums[r * C + c];
      if (!(mx > cur)) { mx = cur; idx = c; }
    }
    out[r] = (int8_t)idx;
  }
}

/* Closed-form softmax over f64 margins (parity unpinned in the reference). */
void oracle_softmax(const double *sums, int64_t rows, int32_t C, double *out) {
  for (int64_t r = 0; r < rows; ++r) {
    double mx = sums[r * C];
    for (int32_t c = 1; c < C; ++c) if (sums[r * C + c] > mx) mx = sums[r * C + c];
    double z = 0;
    for (int32_t c = 0; c < C; ++c) { out[r * C + c] = exp(sums[r * C + c] - mx); z += out[r * C + c]; }
    for (int32_t c = 0; c < C; ++c) out[r * C + c] /= z;
  }
}

/*
 * Multithreaded CPU path used as the reported CPU baseline: the batch is
 * split evenly over `threads` cores and each chunk is processed one tree at a
 * time, rows inner (ReorderTiledTreesByDepth.cpp:387-398:
 * result[r] = initial; for t: result[r] += leaf_t, f32 accumulation as in the
 * generated code).  Tile size 1.  tree_order gives the depth-sorted order.
 */
void oracle_predict_tree_outer(const oracle_forest_t *f, const float *x,
                               int64_t rows, float *out,
                               const int32_t *tree_order, int32_t threads) {
  const int32_t T = f->num_trees, F = f->num_features;
  if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int32_t k = 0; k < threads; ++k) {
    int64_t lo = rows * k / threads, hi = rows * (k + 1) / threads;
    for (int64_t r = lo; r < hi; ++r) out[r] = (float)f->initial_value;
    for (int32_t i = 0; i < T; ++i) {
      int32_t t = tree_order ? tree_order[i] : i;
      const int64_t base = f->tree_offsets[t];
      for (int64_t r = lo; r < hi; ++r) {
        int32_t n = walk_tree_f32(f, t, x + r * F, NULL);
        out[r] += (float)f->threshold[base + n];
      }
    }
    if (f->transform == 1)
      for (int64_t r = lo; r < hi; ++r) out[r] = 1.0f / (1.0f + expf(-out[r]));
  }
}

int32_t oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

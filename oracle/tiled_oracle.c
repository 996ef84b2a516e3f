/*
 * Tiled CPU walk: restatement of the reference's vectorised CPU path.  TEST INFRASTRUCTURE ONLY
 * (checker for the tiled-walk invariant and the CPU baseline of the benchmark; never part of the
 * product library).
 *
 * Reference code followed (paths relative to the reference checkout):
 *   src/mlir/UniformTilingTransformation.cpp:148-195   a tile = up to T connected internal nodes taken
 *       breadth first (left before right) from the first untiled node met going down the tree;
 *       leaves are never members of a tile
 *   docs/TileShapesAndLUT/TileShapesAndLUT.md:23-27     nodes of a tile are in level order; the children
 *       of a tile are numbered left to right
 *   src/utils/TreeTilingUtils.cpp:1932-2018             LUT[shape][outcome bits] -> child number, a set
 *       bit meaning "predicate true, go left"
 *   src/mlir/CodeGenStateMachine.cpp:284-506            tile step: gather T features, T compares,
 *       outcome bits with node 0 in the least significant bit (UseBitcastForComparisonOutcome,
 *       src/mlir/Dialect.cpp:19), child = LUT[shape][bits]
 *   src/mlir/Representations.cpp:1491-1497, :1678-1690  sparse layout: next = childBase + child; an
 *       index at or beyond the tree's tile count is a leaf, value leaves[index - tiles]
 *   src/utils/TreeTilingUtils.cpp:1290-1310             a leaf whose siblings are not all leaves gets an
 *       extra hop tile so that the children of every tile are consecutive
 *   src/utils/TreeTilingUtils.cpp:1614-1720             short tiles are padded to T nodes; here the pad
 *       slots hold a comparison whose outcome bits are don't-cares of the shape's LUT row, which
 *       reaches the same leaf as the reference's spliced-in dummy nodes
 *   src/mlir/ReorderTiledTreesByDepth.cpp:387-398        batch split over cores, one tree at a time,
 *       rows inner, f32 accumulation (configs/b512_t8_uniform_pipeline8_noPar.json: tile size 8)
 *
 * Pinned by tests/test_oracle.py: leaf reached == the scalar oracle's leaf on the reference's fixtures
 * and on random trees for T in {1,2,3,4,8}; number of tile shapes of size T == Catalan(T)
 * (docs/TileShapesAndLUT/TileShapesAndLUT.md:15-19); the documented LUT example (left chain of three
 * nodes: outcome 110 -> child 1, 111 -> child 0, 0xx -> child 3, :46).  The numbering of shapes is
 * this file's own (the reference's numbering is not needed for parity).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__x86_64__)
#include <immintrin.h>
#endif

#define MAX_TILE 8

typedef struct {
  int32_t n;                               /* internal nodes in the tile (0: hop tile) */
  int32_t left[MAX_TILE], right[MAX_TILE]; /* tile-local slot of the child, or -(child number + 1) */
} tile_shape_t;

typedef struct {
  int32_t tile_size;
  int32_t num_trees;
  int32_t num_features;
  int32_t num_shapes;
  int64_t total_tiles, total_leaves;
  int64_t *tile_begin;  /* [num_trees + 1] */
  int64_t *leaf_begin;  /* [num_trees + 1] */
  float *threshold;     /* [tiles][T] */
  int32_t *feature;     /* [tiles][T] */
  int32_t *shape;       /* [tiles] */
  int32_t *child_base;  /* [tiles] tree-local index of child 0; >= the tree's tile count: a leaf */
  float *leaf_value;    /* [leaves] */
  int32_t *leaf_node;   /* [leaves] node id of the leaf in the original tree */
  int8_t *lut;          /* [num_shapes][1 << T] */
  int32_t *shape_nodes; /* [num_shapes] internal nodes of each shape (0: hop tile) */
} tiled_forest_t;

/* Child number reached from the tile root for one outcome word (bit i = node i's predicate, 1 = left). */
static int shape_exit(const tile_shape_t *s, uint32_t bits) {
  if (s->n == 0) return 0; /* hop tile: a single child whatever the outcomes */
  int n = 0;
  for (;;) {
    const int next = ((bits >> n) & 1u) ? s->left[n] : s->right[n];
    if (next < 0) return -next - 1;
    n = next;
  }
}

static int shape_equal(const tile_shape_t *a, const tile_shape_t *b) {
  if (a->n != b->n) return 0;
  for (int i = 0; i < a->n; ++i)
    if (a->left[i] != b->left[i] || a->right[i] != b->right[i]) return 0;
  return 1;
}

typedef struct {
  tile_shape_t *shapes;
  int32_t count, capacity;
} shape_table_t;

static int32_t intern_shape(shape_table_t *t, const tile_shape_t *s) {
  for (int32_t i = 0; i < t->count; ++i)
    if (shape_equal(&t->shapes[i], s)) return i;
  if (t->count == t->capacity) {
    t->capacity = t->capacity ? t->capacity * 2 : 64;
    t->shapes = (tile_shape_t *)realloc(t->shapes, sizeof(tile_shape_t) * (size_t)t->capacity);
  }
  t->shapes[t->count] = *s;
  return t->count++;
}

static int is_leaf(const int32_t *L, const int32_t *R, int32_t n) { return L[n] == -1 && R[n] == -1; }

/* UniformTilingTransformation.cpp:148-168: breadth first over internal nodes only, at most T. */
static int gather_tile(const int32_t *L, const int32_t *R, int32_t root, int T, int32_t *members) {
  int32_t queue[2 * MAX_TILE + 2];
  int head = 0, tail = 0, n = 0;
  queue[tail++] = root;
  while (head < tail && n < T) {
    const int32_t node = queue[head++];
    members[n++] = node;
    if (tail < 2 * MAX_TILE && !is_leaf(L, R, L[node])) queue[tail++] = L[node];
    if (tail < 2 * MAX_TILE && !is_leaf(L, R, R[node])) queue[tail++] = R[node];
  }
  return n;
}

/* Shape of a tile (children as tile-local slots) and its exits in left-to-right order. */
static int describe_tile(const int32_t *L, const int32_t *R, const int32_t *members, int m, tile_shape_t *s,
                         int32_t *exit_node) {
  s->n = m;
  for (int i = 0; i < m; ++i) {
    s->left[i] = s->right[i] = -1;
    for (int j = 0; j < m; ++j) {
      if (members[j] == L[members[i]]) s->left[i] = j;
      if (members[j] == R[members[i]]) s->right[i] = j;
    }
  }
  /* in-order walk of the tile: every missing child is the next exit */
  int ne = 0, sp = 0;
  int32_t stack[2 * MAX_TILE + 2];
  stack[sp++] = 0;
  while (sp > 0) {
    const int32_t item = stack[--sp];
    const int32_t slot = item >> 1;
    if ((item & 1) == 0) {
      stack[sp++] = slot * 2 + 1; /* right side later */
      if (s->left[slot] >= 0) stack[sp++] = s->left[slot] * 2;
      else { exit_node[ne] = L[members[slot]]; s->left[slot] = -(ne++) - 1; }
    } else {
      if (s->right[slot] >= 0) stack[sp++] = s->right[slot] * 2;
      else { exit_node[ne] = R[members[slot]]; s->right[slot] = -(ne++) - 1; }
    }
  }
  return ne;
}

void tiled_forest_free(tiled_forest_t *f) {
  if (!f) return;
  free(f->tile_begin); free(f->leaf_begin); free(f->threshold); free(f->feature); free(f->shape);
  free(f->child_base); free(f->leaf_value); free(f->leaf_node); free(f->lut); free(f->shape_nodes); free(f);
}

/*
 * Builds the tiled, sparse representation of a forest given as flat arrays (layout of
 * oracle_forest_t in forest_oracle.c; the comparison must be "x < threshold goes left").
 */
tiled_forest_t *tiled_forest_build(int32_t num_trees, int32_t num_features, const int64_t *tree_offsets,
                                   const double *threshold, const int32_t *feature, const int32_t *left,
                                   const int32_t *right, int32_t tile_size) {
  if (tile_size < 1 || tile_size > MAX_TILE) return NULL;
  const int T = tile_size;
  tiled_forest_t *f = (tiled_forest_t *)calloc(1, sizeof(tiled_forest_t));
  f->tile_size = T; f->num_trees = num_trees; f->num_features = num_features;
  f->tile_begin = (int64_t *)calloc((size_t)num_trees + 1, sizeof(int64_t));
  f->leaf_begin = (int64_t *)calloc((size_t)num_trees + 1, sizeof(int64_t));
  /* bounds: tiles <= internal nodes + hop tiles <= nodes; leaves <= nodes */
  const size_t cap = (size_t)tree_offsets[num_trees] + (size_t)num_trees + 1;
  f->threshold = (float *)calloc(cap * T, sizeof(float));
  f->feature = (int32_t *)calloc(cap * T, sizeof(int32_t));
  f->shape = (int32_t *)calloc(cap, sizeof(int32_t));
  f->child_base = (int32_t *)calloc(cap, sizeof(int32_t));
  f->leaf_value = (float *)calloc(cap, sizeof(float));
  f->leaf_node = (int32_t *)calloc(cap, sizeof(int32_t));
  shape_table_t table = {0};
  tile_shape_t hop;
  memset(&hop, 0, sizeof(hop));
  const int32_t hop_shape = intern_shape(&table, &hop);

  int32_t *queue = NULL; /* per tile of the tree: root node, or -(leaf node) - 1 for a hop tile */
  for (int32_t t = 0; t < num_trees; ++t) {
    const int64_t base = tree_offsets[t];
    const int32_t n = (int32_t)(tree_offsets[t + 1] - base);
    const int32_t *L = left + base, *R = right + base;
    queue = (int32_t *)realloc(queue, sizeof(int32_t) * ((size_t)n + 1));
    const int64_t tile_base = f->total_tiles, leaf_base = f->total_leaves;
    int32_t tiles = 0, leaves = 0, head = 0;
    if (is_leaf(L, R, 0)) { /* the whole tree is one leaf */
      f->leaf_value[leaf_base] = (float)threshold[base];
      f->leaf_node[leaf_base] = 0;
      leaves = 1;
    } else {
      queue[tiles++] = 0;
    }
    /* Breadth first over the tile hierarchy: the children of a tile get consecutive indices. */
    while (head < tiles) {
      const int64_t ti = tile_base + head;
      const int32_t entry = queue[head];
      if (entry < 0) { /* hop tile in front of a leaf */
        const int32_t leaf = -entry - 1;
        f->shape[ti] = hop_shape;
        f->child_base[ti] = -(leaves + 1); /* leaf reference, resolved below */
        f->leaf_value[leaf_base + leaves] = (float)threshold[base + leaf];
        f->leaf_node[leaf_base + leaves] = leaf;
        ++leaves;
        ++head;
        continue;
      }
      int32_t members[MAX_TILE], exit_node[MAX_TILE + 1];
      const int m = gather_tile(L, R, entry, T, members);
      tile_shape_t s;
      const int ne = describe_tile(L, R, members, m, &s, exit_node);
      f->shape[ti] = intern_shape(&table, &s);
      for (int i = 0; i < m; ++i) {
        f->threshold[ti * T + i] = (float)threshold[base + members[i]];
        f->feature[ti * T + i] = feature[base + members[i]];
      }
      int all_leaves = 1;
      for (int e = 0; e < ne; ++e) all_leaves &= is_leaf(L, R, exit_node[e]);
      if (all_leaves) {
        f->child_base[ti] = -(leaves + 1);
        for (int e = 0; e < ne; ++e) {
          f->leaf_value[leaf_base + leaves] = (float)threshold[base + exit_node[e]];
          f->leaf_node[leaf_base + leaves] = exit_node[e];
          ++leaves;
        }
      } else {
        f->child_base[ti] = tiles;
        for (int e = 0; e < ne; ++e)
          queue[tiles++] = is_leaf(L, R, exit_node[e]) ? -exit_node[e] - 1 : exit_node[e];
      }
      ++head;
    }
    for (int32_t q = 0; q < tiles; ++q) /* leaf references: index >= tile count means leaf */
      if (f->child_base[tile_base + q] < 0) f->child_base[tile_base + q] = tiles + (-f->child_base[tile_base + q] - 1);
    f->total_tiles += tiles;
    f->total_leaves += leaves;
    f->tile_begin[t + 1] = f->total_tiles;
    f->leaf_begin[t + 1] = f->total_leaves;
  }
  free(queue);

  f->num_shapes = table.count;
  f->lut = (int8_t *)malloc((size_t)table.count << T);
  f->shape_nodes = (int32_t *)malloc(sizeof(int32_t) * (size_t)table.count);
  for (int32_t s = 0; s < table.count; ++s) {
    f->shape_nodes[s] = table.shapes[s].n;
    for (uint32_t bits = 0; bits < (1u << T); ++bits)
      f->lut[((size_t)s << T) + bits] = (int8_t)shape_exit(&table.shapes[s], bits);
  }
  free(table.shapes);
  return f;
}

int64_t tiled_forest_num_tiles(const tiled_forest_t *f) { return f->total_tiles; }
int32_t tiled_forest_num_shapes(const tiled_forest_t *f) { return f->num_shapes; }

/* One tile step, scalar form: outcome bit i = (x[feature_i] < threshold_i). */
static inline uint32_t tile_outcomes(const tiled_forest_t *f, int64_t ti, const float *row) {
  const int T = f->tile_size;
  const float *thr = f->threshold + ti * T;
  const int32_t *fi = f->feature + ti * T;
  uint32_t bits = 0;
  for (int i = 0; i < T; ++i) bits |= (uint32_t)(row[fi[i]] < thr[i]) << i;
  return bits;
}

#if defined(__x86_64__)
/* Tile size 8: one AVX2 gather, one compare, one movemask (the vector form of the reference). */
__attribute__((target("avx2"))) static inline uint32_t tile_outcomes8_avx2(const tiled_forest_t *f, int64_t ti,
                                                                           const float *row) {
  const __m256i idx = _mm256_loadu_si256((const __m256i *)(f->feature + ti * 8));
  const __m256 x = _mm256_i32gather_ps(row, idx, 4);
  const __m256 thr = _mm256_loadu_ps(f->threshold + ti * 8);
  return (uint32_t)_mm256_movemask_ps(_mm256_cmp_ps(x, thr, _CMP_LT_OQ));
}
#endif

static inline int32_t walk_tiled(const tiled_forest_t *f, int32_t t, const float *row, int use_avx2) {
  const int64_t tile_base = f->tile_begin[t];
  const int32_t tiles = (int32_t)(f->tile_begin[t + 1] - tile_base);
  const int T = f->tile_size;
  int32_t cur = 0;
  while (cur < tiles) {
    const int64_t ti = tile_base + cur;
    uint32_t bits;
#if defined(__x86_64__)
    if (use_avx2) bits = tile_outcomes8_avx2(f, ti, row);
    else
#endif
      bits = tile_outcomes(f, ti, row);
    cur = f->child_base[ti] + f->lut[((size_t)f->shape[ti] << T) + bits];
  }
  return cur - tiles; /* leaf index inside the tree */
}

static int have_avx2(const tiled_forest_t *f) {
#if defined(__x86_64__)
  return f->tile_size == 8 && __builtin_cpu_supports("avx2");
#else
  (void)f;
  return 0;
#endif
}

/* Original node id of the leaf every (row, tree) reaches through the tiled walk. */
void tiled_leaf_ids(const tiled_forest_t *f, const float *x, int64_t rows, int32_t *leaf_ids, int32_t threads) {
  const int32_t NT = f->num_trees, F = f->num_features;
  const int avx = have_avx2(f);
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
  for (int64_t r = 0; r < rows; ++r)
    for (int32_t t = 0; t < NT; ++t)
      leaf_ids[r * NT + t] = f->leaf_node[f->leaf_begin[t] + walk_tiled(f, t, x + r * F, avx)];
}

/*
 * The multithreaded CPU schedule (ReorderTiledTreesByDepth.cpp:387-398): the batch is cut into
 * `threads` equal chunks; inside a chunk: result[r] = initial; for each tree (given order):
 * for each row: result[r] += leaf; then the sigmoid when asked.  f32 accumulation.
 */
void tiled_predict_tree_outer(const tiled_forest_t *f, const float *x, int64_t rows, float initial_value,
                              int32_t sigmoid, float *out, const int32_t *tree_order, int32_t threads) {
  const int32_t NT = f->num_trees, F = f->num_features;
  const int avx = have_avx2(f);
  if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int32_t k = 0; k < threads; ++k) {
    const int64_t lo = rows * k / threads, hi = rows * (k + 1) / threads;
    for (int64_t r = lo; r < hi; ++r) out[r] = initial_value;
    for (int32_t i = 0; i < NT; ++i) {
      const int32_t t = tree_order ? tree_order[i] : i;
      const float *leaves = f->leaf_value + f->leaf_begin[t];
      for (int64_t r = lo; r < hi; ++r) out[r] += leaves[walk_tiled(f, t, x + r * F, avx)];
    }
    if (sigmoid)
      for (int64_t r = lo; r < hi; ++r) out[r] = 1.0f / (1.0f + expf(-out[r]));
  }
}

/*
 * The same schedule for a multiclass forest: every chunk keeps f32 class sums [rows][C], each filled with the
 * initial value before the trees are added (src/reduction/LowerReduceOps.cpp:1459-1470), tree t adds its leaf to
 * class class_id[t] (GenerateMultiClassAccumulate, src/mlir/LowerToMidLevelIR.cpp:405-429), and the class id is
 * the generated code's arg-max: running maximum from -inf / class 0, replaced unless `max > cur`, so exact ties go
 * to the larger class id (LowerReduceOps.cpp:148-187).  `sums` may be NULL; `out_class` takes the ids as int8.
 */
void tiled_predict_tree_outer_multiclass(const tiled_forest_t *f, const float *x, int64_t rows, float initial_value,
                                         int32_t num_classes, const int32_t *class_id, int8_t *out_class, float *sums,
                                         const int32_t *tree_order, int32_t threads) {
  const int32_t NT = f->num_trees, F = f->num_features, C = num_classes;
  const int avx = have_avx2(f);
  if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int32_t k = 0; k < threads; ++k) {
    const int64_t lo = rows * k / threads, hi = rows * (k + 1) / threads;
    if (hi <= lo) continue;
    float *acc = sums ? sums + lo * C : (float *)malloc((size_t)(hi - lo) * (size_t)C * sizeof(float));
    for (int64_t i = 0; i < (hi - lo) * C; ++i) acc[i] = initial_value;
    for (int32_t i = 0; i < NT; ++i) {
      const int32_t t = tree_order ? tree_order[i] : i;
      const float *leaves = f->leaf_value + f->leaf_begin[t];
      const int32_t c = class_id[t];
      for (int64_t r = lo; r < hi; ++r) acc[(r - lo) * C + c] += leaves[walk_tiled(f, t, x + r * F, avx)];
    }
    for (int64_t r = lo; r < hi; ++r) {
      float mx = -INFINITY;
      int32_t idx = 0;
      for (int32_t c = 0; c < C; ++c) {
        const float cur = acc[(r - lo) * C + c];
        if (!(mx > cur)) { mx = cur; idx = c; }
      }
      out_class[r] = (int8_t)idx;
    }
    if (!sums) free(acc);
  }
}

/* LUT row of an explicitly given shape (for the documented known-answer checks). */
void tiled_lut_for_shape(int32_t n, const int32_t *left_slot, const int32_t *right_slot, int32_t tile_size,
                         int8_t *lut_row) {
  tile_shape_t s;
  memset(&s, 0, sizeof(s));
  s.n = n;
  int exits = 0;
  /* children given as slot (>= 0) or -1; exits are numbered left to right as in describe_tile */
  int32_t stack[2 * MAX_TILE + 2];
  int sp = 0;
  for (int i = 0; i < n; ++i) { s.left[i] = left_slot[i]; s.right[i] = right_slot[i]; }
  stack[sp++] = 0;
  while (sp > 0) {
    const int32_t item = stack[--sp];
    const int32_t slot = item >> 1;
    if ((item & 1) == 0) {
      stack[sp++] = slot * 2 + 1;
      if (s.left[slot] >= 0) stack[sp++] = s.left[slot] * 2;
      else s.left[slot] = -(exits++) - 1;
    } else {
      if (s.right[slot] >= 0) stack[sp++] = s.right[slot] * 2;
      else s.right[slot] = -(exits++) - 1;
    }
  }
  for (uint32_t bits = 0; bits < (1u << tile_size); ++bits) lut_row[bits] = (int8_t)shape_exit(&s, bits);
}

/* How many of the forest's distinct tile shapes have exactly n internal nodes. */
int32_t tiled_forest_shapes_with_nodes(const tiled_forest_t *f, int32_t n) {
  int32_t count = 0;
  for (int32_t s = 0; s < f->num_shapes; ++s) count += f->shape_nodes[s] == n;
  return count;
}

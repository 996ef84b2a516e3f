"""ctypes binding of the C oracle (oracle/forest_oracle.c).  TEST INFRASTRUCTURE ONLY.

Nothing in the product imports this module: it is the checker for tests/,
the smoke check and the benchmark's CPU-baseline leg.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libtbref.so")


class _CForest(ctypes.Structure):
    _fields_ = [("num_trees", ctypes.c_int32), ("num_features", ctypes.c_int32),
                ("num_classes", ctypes.c_int32), ("transform", ctypes.c_int32),
                ("predicate", ctypes.c_int32), ("initial_value", ctypes.c_double),
                ("tree_offsets", ctypes.c_void_p), ("threshold", ctypes.c_void_p),
                ("feature", ctypes.c_void_p), ("left", ctypes.c_void_p),
                ("right", ctypes.c_void_p), ("class_id", ctypes.c_void_p)]


def build(force=False):
    """Compile the C oracle (and oracle/_ref when the reference checkout is present)."""
    args = ["make", "-s", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(args, check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_total_steps.restype = ctypes.c_int64
        _lib.oracle_max_threads.restype = ctypes.c_int32
    return _lib


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def c_forest(forest):
    """Returns (struct, keepalive list)."""
    keep = [np.ascontiguousarray(forest.tree_offsets, dtype=np.int64),
            np.ascontiguousarray(forest.threshold, dtype=np.float64),
            np.ascontiguousarray(forest.feature, dtype=np.int32),
            np.ascontiguousarray(forest.left, dtype=np.int32),
            np.ascontiguousarray(forest.right, dtype=np.int32),
            np.ascontiguousarray(forest.class_id, dtype=np.int32)]
    cf = _CForest(forest.num_trees, forest.num_features, forest.num_classes, forest.transform,
                  forest.predicate, forest.initial_value, *[a.ctypes.data for a in keep])
    return cf, keep


def max_threads():
    return int(lib().oracle_max_threads())


def leaf_ids(forest, x, want_path_len=False, threads=0):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows = x.shape[0]
    cf, keep = c_forest(forest)
    ids = np.empty((rows, forest.num_trees), dtype=np.int32)
    plen = np.empty((rows, forest.num_trees), dtype=np.int32) if want_path_len else None
    lib().oracle_leaf_ids(ctypes.byref(cf), _ptr(x), ctypes.c_int64(rows), _ptr(ids),
                          _ptr(plen) if want_path_len else None,
                          ctypes.c_int32(threads or max_threads()))
    return (ids, plen) if want_path_len else ids


def total_steps(forest, x, threads=0):
    x = np.ascontiguousarray(x, dtype=np.float32)
    cf, keep = c_forest(forest)
    return int(lib().oracle_total_steps(ctypes.byref(cf), _ptr(x), ctypes.c_int64(x.shape[0]),
                                        ctypes.c_int32(threads or max_threads())))


def predict(forest, x, threads=0):
    """Returns (pred f32[rows], margins f64[rows] or f64[rows][C])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows = x.shape[0]
    cf, keep = c_forest(forest)
    C = max(1, forest.num_classes)
    pred = np.empty(rows, dtype=np.float32)
    sums = np.empty((rows, C), dtype=np.float64)
    lib().oracle_predict_f32(ctypes.byref(cf), _ptr(x), ctypes.c_int64(rows), _ptr(pred), _ptr(sums),
                             ctypes.c_int32(threads or max_threads()))
    return pred, (sums[:, 0] if forest.num_classes == 0 else sums)


def predict_f64(forest, x):
    x = np.ascontiguousarray(x, dtype=np.float64)
    cf, keep = c_forest(forest)
    pred = np.empty(x.shape[0], dtype=np.float64)
    lib().oracle_predict_f64(ctypes.byref(cf), _ptr(x), ctypes.c_int64(x.shape[0]), _ptr(pred))
    return pred


def argmax_generated(sums_f32):
    s = np.ascontiguousarray(sums_f32, dtype=np.float32)
    out = np.empty(s.shape[0], dtype=np.int8)
    lib().oracle_argmax_generated(_ptr(s), ctypes.c_int64(s.shape[0]), ctypes.c_int32(s.shape[1]), _ptr(out))
    return out


def softmax(sums_f64):
    s = np.ascontiguousarray(sums_f64, dtype=np.float64)
    out = np.empty_like(s)
    lib().oracle_softmax(_ptr(s), ctypes.c_int64(s.shape[0]), ctypes.c_int32(s.shape[1]), _ptr(out))
    return out


def predict_tree_outer(forest, x, tree_order=None, threads=0):
    """The multithreaded one-tree-at-a-time CPU schedule (f32 accumulation)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    cf, keep = c_forest(forest)
    out = np.empty(x.shape[0], dtype=np.float32)
    order = None if tree_order is None else np.ascontiguousarray(tree_order, dtype=np.int32)
    lib().oracle_predict_tree_outer(ctypes.byref(cf), _ptr(x), ctypes.c_int64(x.shape[0]), _ptr(out),
                                    _ptr(order) if order is not None else None,
                                    ctypes.c_int32(threads or max_threads()))
    return out


# --------------------------------------------------------------------------
# tiled CPU walk (oracle/tiled_oracle.c)
# --------------------------------------------------------------------------
class TiledForest:
    """Uniformly tiled, sparse-layout forest with its LUT (tile size 1..8)."""

    def __init__(self, forest, tile_size):
        assert forest.predicate == 0, "the tiled walk takes 'x < threshold goes left' forests"
        L = lib()
        L.tiled_forest_build.restype = ctypes.c_void_p
        L.tiled_forest_num_tiles.restype = ctypes.c_int64
        self._L = L
        self.forest = forest
        self.tile_size = tile_size
        keep = c_forest(forest)[1]
        self.h = ctypes.c_void_p(L.tiled_forest_build(
            ctypes.c_int32(forest.num_trees), ctypes.c_int32(forest.num_features), _ptr(keep[0]), _ptr(keep[1]),
            _ptr(keep[2]), _ptr(keep[3]), _ptr(keep[4]), ctypes.c_int32(tile_size)))
        assert self.h, "tile size must be in 1..8"

    def __del__(self):
        try:
            self._L.tiled_forest_free(self.h)
        except Exception:
            pass

    def num_tiles(self):
        return int(self._L.tiled_forest_num_tiles(self.h))

    def num_shapes(self):
        return int(self._L.tiled_forest_num_shapes(self.h))

    def shapes_with_nodes(self, n):
        return int(self._L.tiled_forest_shapes_with_nodes(self.h, ctypes.c_int32(n)))

    def leaf_ids(self, x, threads=0):
        x = np.ascontiguousarray(x, dtype=np.float32)
        ids = np.empty((x.shape[0], self.forest.num_trees), dtype=np.int32)
        self._L.tiled_leaf_ids(self.h, _ptr(x), ctypes.c_int64(x.shape[0]), _ptr(ids),
                               ctypes.c_int32(threads or max_threads()))
        return ids

    def predict_tree_outer(self, x, tree_order=None, threads=0):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape[0], dtype=np.float32)
        order = None if tree_order is None else np.ascontiguousarray(tree_order, dtype=np.int32)
        self._L.tiled_predict_tree_outer(self.h, _ptr(x), ctypes.c_int64(x.shape[0]),
                                         ctypes.c_float(self.forest.initial_value),
                                         ctypes.c_int32(1 if self.forest.transform == 1 else 0), _ptr(out),
                                         _ptr(order) if order is not None else None,
                                         ctypes.c_int32(threads or max_threads()))
        return out


    def predict_tree_outer_multiclass(self, x, tree_order=None, threads=0):
        """Class ids (int8) and f32 class sums of the multithreaded tree-at-a-time schedule on a multiclass forest."""
        assert self.forest.num_classes > 0
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape[0], dtype=np.int8)
        sums = np.empty((x.shape[0], self.forest.num_classes), dtype=np.float32)
        order = None if tree_order is None else np.ascontiguousarray(tree_order, dtype=np.int32)
        class_id = np.ascontiguousarray(self.forest.class_id, dtype=np.int32)
        self._L.tiled_predict_tree_outer_multiclass(self.h, _ptr(x), ctypes.c_int64(x.shape[0]),
                                                    ctypes.c_float(self.forest.initial_value),
                                                    ctypes.c_int32(self.forest.num_classes), _ptr(class_id), _ptr(out),
                                                    _ptr(sums), _ptr(order) if order is not None else None,
                                                    ctypes.c_int32(threads or max_threads()))
        return out, sums


def lut_for_shape(left_slot, right_slot, tile_size):
    """LUT row (2^tile_size entries) of a tile whose nodes (level order) have the given children slots (-1: exit)."""
    l = np.ascontiguousarray(left_slot, dtype=np.int32)
    r = np.ascontiguousarray(right_slot, dtype=np.int32)
    row = np.empty(1 << tile_size, dtype=np.int8)
    lib().tiled_lut_for_shape(ctypes.c_int32(len(l)), _ptr(l), _ptr(r), ctypes.c_int32(tile_size), _ptr(row))
    return row


# --------------------------------------------------------------------------
# oracle/_ref: the reference's own header (DecisionForest.h) behind a C driver
# --------------------------------------------------------------------------
_ref = None


def ref_available():
    return os.path.exists(_REF_PATH)


def ref_lib():
    global _ref
    if _ref is None:
        _ref = ctypes.CDLL(_REF_PATH)
        _ref.tbref_create.restype = ctypes.c_void_p
    return _ref


class RefForest:
    """DecisionForest built through the reference's NewTree/NewNode/SetNode* API."""

    def __init__(self, forest):
        L = ref_lib()
        self._L = L
        self.forest = forest
        self.h = ctypes.c_void_p(L.tbref_create(ctypes.c_double(forest.initial_value),
                                                ctypes.c_int32(forest.transform),
                                                ctypes.c_int32(forest.num_classes)))
        for t in range(forest.num_trees):
            thr, feat, left, right = forest.tree(t)
            thr = np.ascontiguousarray(thr, dtype=np.float64)
            feat = np.ascontiguousarray(feat, dtype=np.int32)
            left = np.ascontiguousarray(left, dtype=np.int32)
            right = np.ascontiguousarray(right, dtype=np.int32)
            L.tbref_add_tree(self.h, ctypes.c_int32(len(thr)), _ptr(thr), _ptr(feat), _ptr(left), _ptr(right),
                             ctypes.c_int32(int(forest.class_id[t])))

    def __del__(self):
        try:
            self._L.tbref_destroy(self.h)
        except Exception:
            pass

    def predict_float(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(x.shape[0], dtype=np.float32)
        self._L.tbref_predict_float(self.h, _ptr(x), ctypes.c_int64(x.shape[0]), ctypes.c_int32(x.shape[1]), _ptr(out))
        return out

    def predict_double(self, x):
        x = np.ascontiguousarray(x, dtype=np.float64)
        out = np.empty(x.shape[0], dtype=np.float64)
        self._L.tbref_predict_double(self.h, _ptr(x), ctypes.c_int64(x.shape[0]), ctypes.c_int32(x.shape[1]), _ptr(out))
        return out

    def tree_values_float(self, x):
        """PredictTree_Float for every (row, tree): the leaf VALUE the reference returns."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty((x.shape[0], self.forest.num_trees), dtype=np.float32)
        self._L.tbref_tree_values_float(self.h, _ptr(x), ctypes.c_int64(x.shape[0]), ctypes.c_int32(x.shape[1]), _ptr(out))
        return out

    def dense_arrays(self, t):
        """GetThresholdArray / GetFeatureIndexArray of tree t (DecisionForest.h:292-315)."""
        n = self._L.tbref_dense_size(self.h, ctypes.c_int32(t))
        thr = np.empty(n, dtype=np.float64)
        idx = np.empty(n, dtype=np.int32)
        self._L.tbref_dense_arrays(self.h, ctypes.c_int32(t), _ptr(thr), _ptr(idx))
        return thr, idx

    def sparse_arrays(self, t):
        """GetSparseThresholdArray / GetSparseFeatureIndexArray / GetChildIndexArray (:595-629)."""
        n = self._L.tbref_sparse_size(self.h, ctypes.c_int32(t))
        thr = np.empty(n, dtype=np.float64)
        idx = np.empty(n, dtype=np.int32)
        child = np.empty(n, dtype=np.int32)
        self._L.tbref_sparse_arrays(self.h, ctypes.c_int32(t), _ptr(thr), _ptr(idx), _ptr(child))
        return thr, idx, child

    def depth(self, t):
        return int(self._L.tbref_tree_depth(self.h, ctypes.c_int32(t)))

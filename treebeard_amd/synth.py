"""Seeded synthetic models and batches for the five benchmark configurations.

Models are written as XGBoost-JSON with the same skeleton the reference's
random-forest writer emits (src/utils/RandomTreeGenerator.cpp:83-167: nodes in
level order, `default_left` all false, root parent 2147483647, leaf value in
`split_conditions`), extended with `objective.name`, `num_class` and
`tree_info` for the classifier configurations.  Every threshold / leaf value is
a float32 printed with `repr`, so `(float)strtod(text)` reproduces it exactly.

Seeds: model 1000+k, quantile sample 2000+k, batch 3000+k for configuration k.
"""
import json
import os

import numpy as np

ROOT_PARENT = 2147483647


class TreeArrays:
    __slots__ = ("left", "right", "parent", "feature", "value")

    def __init__(self):
        self.left, self.right, self.parent, self.feature, self.value = [], [], [], [], []


def _grow_tree(rng, max_depth, split_prob, draw_split, draw_leaf, force_root=True):
    """Level-order growth.  split_prob(depth, side) -> probability that a
    candidate node at `depth` (side 0 = left child, 1 = right child, -1 = root)
    becomes an internal node."""
    t = TreeArrays()
    t.left.append(-1); t.right.append(-1); t.parent.append(ROOT_PARENT); t.feature.append(0); t.value.append(0.0)
    queue = [(0, 0, -1)]
    head = 0
    while head < len(queue):
        nid, depth, side = queue[head]
        head += 1
        split = depth < max_depth and ((force_root and depth == 0) or rng.random() < split_prob(depth, side))
        if split:
            f, thr = draw_split()
            t.feature[nid] = int(f)
            t.value[nid] = float(np.float32(thr))
            for s in (0, 1):
                cid = len(t.left)
                t.left.append(-1); t.right.append(-1); t.parent.append(nid); t.feature.append(0); t.value.append(0.0)
                if s == 0:
                    t.left[nid] = cid
                else:
                    t.right[nid] = cid
                queue.append((cid, depth + 1, s))
        else:
            t.value[nid] = float(np.float32(draw_leaf()))
    return t


def write_xgboost_json(path, trees, num_features, objective="reg:squarederror", base_score="5E-1",
                       num_class=0, tree_info=None):
    tree_info = list(tree_info) if tree_info is not None else [0] * len(trees)
    tj = []
    for i, t in enumerate(trees):
        n = len(t.left)
        zeros = [0.0] * n
        tj.append({
            "base_weights": zeros, "categories": [], "categories_nodes": [], "categories_segments": [],
            "categories_sizes": [], "default_left": [False] * n, "id": i,
            "left_children": t.left, "loss_changes": zeros, "parents": t.parent,
            "right_children": t.right, "split_conditions": t.value, "split_indices": t.feature,
            "split_type": [0] * n, "sum_hessian": zeros,
            "tree_param": {"num_deleted": "0", "num_feature": str(num_features), "num_nodes": str(n),
                           "size_leaf_vector": "0"}})
    doc = {"learner": {
        "attributes": {}, "feature_names": [], "feature_types": ["float"] * num_features,
        "gradient_booster": {"model": {"gbtree_model_param": {"num_trees": str(len(trees)), "size_leaf_vector": "0"},
                                       "tree_info": tree_info, "trees": tj}, "name": "gbtree"},
        "learner_model_param": {"base_score": base_score, "num_class": str(num_class),
                                "num_feature": str(num_features)},
        "objective": {"name": objective, "reg_loss_param": {"scale_pos_weight": "1"}}},
        "version": [1, 4, 0]}
    tmp = str(path) + ".tmp"
    with open(tmp, "w") as fh:
        json.dump(doc, fh)
    os.replace(tmp, path)


def _quantile_table(seed, num_features, rows=100_000, levels=4096):
    """Per-feature empirical quantiles of a seeded N(0,1) sample."""
    rng = np.random.Generator(np.random.PCG64(seed))
    sample = rng.standard_normal((rows, num_features), dtype=np.float32)
    qs = np.linspace(0.0, 1.0, levels)
    return np.quantile(sample, qs, axis=0).astype(np.float32), sample


class Config:
    def __init__(self, k, name, num_features, batch, objective, num_class=0, sweep=()):
        self.k, self.name, self.num_features, self.batch = k, name, num_features, batch
        self.objective, self.num_class, self.sweep = objective, num_class, tuple(sweep)

    def model(self, path):
        trees, info = _MODEL_BUILDERS[self.k](self)
        write_xgboost_json(path, trees, self.num_features, objective=self.objective, num_class=self.num_class,
                           tree_info=info)
        return path

    def batch_rows(self, rows=None, seed_offset=0):
        rows = self.batch if rows is None else rows
        rng = np.random.Generator(np.random.PCG64(3000 + self.k + 7919 * seed_offset))
        return _BATCH_BUILDERS[self.k](self, rng, rows)


def _model_c1(cfg):
    rng = np.random.Generator(np.random.PCG64(1001))
    trees = [_grow_tree(rng, 6, lambda d, s: 1.0,
                        lambda: (rng.integers(0, 8), rng.random()),
                        lambda: rng.normal(0.0, 0.1)) for _ in range(100)]
    return trees, None


def _model_c2(cfg):
    rng = np.random.Generator(np.random.PCG64(1002))
    qt, _ = _quantile_table(2002, 28)

    def split():
        f = rng.integers(0, 28)
        return f, qt[rng.integers(0, qt.shape[0]), f]
    trees = [_grow_tree(rng, 8, lambda d, s: 0.8, split, lambda: rng.normal(0.0, 0.05)) for _ in range(1000)]
    return trees, None


def _model_c3(cfg):
    rng = np.random.Generator(np.random.PCG64(1003))
    qt, _ = _quantile_table(2003, 10)

    def split():
        f = rng.integers(0, 54)
        if f < 10:
            return f, qt[rng.integers(0, qt.shape[0]), f]
        return f, 0.5
    trees = [_grow_tree(rng, 6, lambda d, s: 1.0, split, lambda: rng.normal(0.0, 0.1)) for _ in range(800)]
    return trees, [t % 8 for t in range(800)]


def _model_c4(cfg):
    rng = np.random.Generator(np.random.PCG64(1004))
    trees = [_grow_tree(rng, 8, lambda d, s: 0.85,
                        lambda: (rng.integers(0, 2000), rng.standard_normal()),
                        lambda: rng.normal(0.0, 0.02)) for _ in range(1000)]
    return trees, None


def _model_c5(cfg):
    rng = np.random.Generator(np.random.PCG64(1005))
    qt, _ = _quantile_table(2005, 90)

    def split():
        f = rng.integers(0, 90)
        return f, qt[rng.integers(0, qt.shape[0]), f]
    trees = [_grow_tree(rng, 12, lambda d, s: 0.9 if s == 0 else 0.3, split, lambda: rng.normal(0.0, 0.05))
             for _ in range(800)]
    return trees, None


def _batch_uniform(cfg, rng, rows):
    return rng.random((rows, cfg.num_features), dtype=np.float32)


def _batch_normal(cfg, rng, rows):
    return rng.standard_normal((rows, cfg.num_features), dtype=np.float32)


def _batch_c3(cfg, rng, rows):
    x = np.empty((rows, 54), dtype=np.float32)
    x[:, :10] = rng.standard_normal((rows, 10), dtype=np.float32)
    x[:, 10:] = (rng.random((rows, 44), dtype=np.float32) < 0.1).astype(np.float32)
    return x


def _batch_c5(cfg, rng, rows):
    """About 80 % of the rows come from a low-shifted population N(-2, 0.5), for
    which `x < threshold` holds at almost every node (left spine); 20 % N(0,1)."""
    x = rng.standard_normal((rows, 90), dtype=np.float32)
    hot = rng.random(rows) < 0.8
    x[hot] = x[hot] * np.float32(0.5) - np.float32(2.0)
    return x


_MODEL_BUILDERS = {1: _model_c1, 2: _model_c2, 3: _model_c3, 4: _model_c4, 5: _model_c5}
_BATCH_BUILDERS = {1: _batch_uniform, 2: _batch_normal, 3: _batch_c3, 4: _batch_normal, 5: _batch_c5}

CONFIGS = {
    1: Config(1, "c1_regression_100x6_f8", 8, 1024, "reg:squarederror"),
    2: Config(2, "c2_binary_1000x8_f28", 28, 1 << 20, "binary:logistic", sweep=(1, 64, 4096, 1 << 16)),
    3: Config(3, "c3_multiclass_800x6_f54", 54, 1 << 20, "multi:softmax", num_class=8),
    4: Config(4, "c4_wide_1000x8_f2000", 2000, 1 << 18, "reg:squarederror"),
    5: Config(5, "c5_skewed_800x12_f90", 90, 1 << 20, "reg:squarederror"),
}


def model_path(k, cache_dir):
    """Writes configuration k's model under cache_dir once and returns its path."""
    os.makedirs(cache_dir, exist_ok=True)
    path = os.path.join(cache_dir, CONFIGS[k].name + ".json")
    if not os.path.exists(path):
        CONFIGS[k].model(path)
    return path

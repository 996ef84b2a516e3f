"""Model loaders for the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Pure-Python restatements of the reference's two front ends; the product's
loaders are the C++ ones inside the runtime library and never import this.

Reference code followed (paths relative to the reference checkout):
  src/json/xgboostparser.h:94-114   TransformBaseScore / GetPredictionTransformType
  src/json/xgboostparser.h:117-145  ConstructForest (base_score, num_class, feature_types)
  src/json/xgboostparser.h:156-174  ConstructTreesFromBooster (tree_info -> class id)
  src/json/xgboostparser.h:177-219  ConstructSingleTree (leaf value = split_conditions[leaf])
  src/json/onnxmodelparser.h:94-177 attribute decoding, compare modes
  src/json/onnxmodelparser.h:220-312 child links, tree starts, leaf weights
  src/json/onnxmodelparser.h:315-374 pre-order node numbering, class id per tree
  src/json/onnx.proto:138-174,196-213,380,441 wire field numbers

Pinned by: the XGBoost golden CSVs the reference ships (tests/golden), the
ONNX abalone fixture and its CSV, and XGBoost-JSON == ONNX forest equality on
models the reference holds in both formats.
"""
import gzip
import json
import math
import struct
from dataclasses import dataclass, field

import numpy as np

IDENTITY, SIGMOID, SOFTMAX = 0, 1, 2
PRED_LT, PRED_GE, PRED_GT, PRED_LE = 0, 1, 2, 3


@dataclass
class Forest:
    num_features: int
    initial_value: float
    transform: int
    num_classes: int
    predicate: int
    tree_offsets: np.ndarray      # int64[T+1]
    threshold: np.ndarray         # float64[N] (f32-representable)
    feature: np.ndarray           # int32[N]
    left: np.ndarray              # int32[N] local index or -1
    right: np.ndarray             # int32[N]
    class_id: np.ndarray          # int32[T]
    meta: dict = field(default_factory=dict)

    @property
    def num_trees(self):
        return len(self.tree_offsets) - 1

    def tree(self, t):
        lo, hi = int(self.tree_offsets[t]), int(self.tree_offsets[t + 1])
        return (self.threshold[lo:hi], self.feature[lo:hi], self.left[lo:hi], self.right[lo:hi])

    def depth(self, t):
        """Number of internal nodes on the longest root-to-leaf path."""
        _, _, l, r = self.tree(t)
        depth = np.zeros(len(l), dtype=np.int32)
        best = 0
        stack = [(0, 0)]
        while stack:
            n, d = stack.pop()
            if l[n] == -1 and r[n] == -1:
                best = max(best, d)
                continue
            stack.append((int(l[n]), d + 1))
            stack.append((int(r[n]), d + 1))
        return best


def _open_text(path):
    path = str(path)
    if path.endswith(".gz"):
        return gzip.open(path, "rt")
    return open(path, "r")


def _open_bytes(path):
    path = str(path)
    if path.endswith(".gz"):
        return gzip.open(path, "rb")
    return open(path, "rb")


def _assemble(trees, **kw):
    offs = np.zeros(len(trees) + 1, dtype=np.int64)
    for i, t in enumerate(trees):
        offs[i + 1] = offs[i] + len(t[0])
    cat = lambda k, dt: (np.concatenate([np.asarray(t[k], dtype=dt) for t in trees])
                         if trees else np.zeros(0, dtype=dt))
    return Forest(tree_offsets=offs, threshold=cat(0, np.float64), feature=cat(1, np.int32),
                  left=cat(2, np.int32), right=cat(3, np.int32), **kw)


def load_xgboost_json(path, threshold_f32=True):
    """xgboostparser.h:117-219."""
    with _open_text(path) as fh:
        doc = json.load(fh)
    learner = doc["learner"]
    base = float(learner["learner_model_param"]["base_score"])        # std::stod
    objective = learner["objective"]["name"]
    if objective == "binary:logistic":
        initial, transform = -math.log(1.0 / base - 1.0), SIGMOID
    elif objective == "reg:squarederror":
        initial, transform = base, IDENTITY
    elif objective == "multi:softmax":
        initial, transform = base, SOFTMAX
    else:
        raise ValueError("Unknown objective type " + objective)
    num_class = int(learner["learner_model_param"]["num_class"])
    num_features = len(learner["feature_types"])
    model = learner["gradient_booster"]["model"]
    trees_json = model["trees"]
    tree_info = model["tree_info"]
    assert int(model["gbtree_model_param"]["num_trees"]) == len(trees_json) == len(tree_info)
    trees = []
    for tj in trees_json:
        n = int(tj["tree_param"]["num_nodes"])
        assert n == len(tj["left_children"]) == len(tj["right_children"]) == len(tj["parents"])
        thr = np.asarray(tj["split_conditions"], dtype=np.float64)
        if threshold_f32:
            thr = thr.astype(np.float32).astype(np.float64)          # get<float>() then widened
        trees.append((thr, tj["split_indices"], tj["left_children"], tj["right_children"]))
    if num_features == 0:
        num_features = int(learner["learner_model_param"]["num_feature"])
    return _assemble(trees, num_features=num_features, initial_value=initial, transform=transform,
                     num_classes=num_class, predicate=PRED_LT,
                     class_id=np.asarray(tree_info, dtype=np.int32),
                     meta={"objective": objective, "base_score": base})


# --------------------------------------------------------------------------
# ONNX: minimal protobuf wire-format reader (no onnx / protoc needed)
# --------------------------------------------------------------------------
def _varint(buf, pos):
    result = shift = 0
    while True:
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7


def _fields(buf):
    pos, end = 0, len(buf)
    while pos < end:
        key, pos = _varint(buf, pos)
        fno, wt = key >> 3, key & 7
        if wt == 0:
            val, pos = _varint(buf, pos)
        elif wt == 1:
            val = buf[pos:pos + 8]; pos += 8
        elif wt == 2:
            ln, pos = _varint(buf, pos)
            val = buf[pos:pos + ln]; pos += ln
        elif wt == 5:
            val = buf[pos:pos + 4]; pos += 4
        else:
            raise ValueError("unsupported wire type %d" % wt)
        yield fno, wt, val


def _sint64(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def _parse_attribute(buf):
    name, f, i, s = None, None, None, None
    floats, ints, strings = [], [], []
    for fno, wt, val in _fields(buf):
        if fno == 1:
            name = bytes(val).decode()
        elif fno == 2:
            f = struct.unpack("<f", val)[0]
        elif fno == 3:
            i = _sint64(val)
        elif fno == 4:
            s = bytes(val)
        elif fno == 7:
            if wt == 5:
                floats.append(struct.unpack("<f", val)[0])
            else:                                   # packed
                floats.extend(np.frombuffer(bytes(val), dtype="<f4").tolist())
        elif fno == 8:
            if wt == 0:
                ints.append(_sint64(val))
            else:                                   # packed varints
                p = 0
                while p < len(val):
                    v, p = _varint(val, p)
                    ints.append(_sint64(v))
        elif fno == 9:
            strings.append(bytes(val))
    return name, dict(f=f, i=i, s=s, floats=floats, ints=ints, strings=strings)


def load_onnx(path, num_features):
    """onnxmodelparser.h:50-374.  num_features comes from the compiler options."""
    with _open_bytes(path) as fh:
        buf = memoryview(fh.read())
    graph = None
    for fno, wt, val in _fields(buf):
        if fno == 7:
            graph = val
    nodes = [val for fno, wt, val in _fields(graph) if fno == 1]
    assert len(nodes) == 1, "Only one node is supported"
    op_type, attrs = None, {}
    for fno, wt, val in _fields(nodes[0]):
        if fno == 4:
            op_type = bytes(val).decode()
        elif fno == 5:
            n, a = _parse_attribute(val)
            attrs[n] = a
    assert op_type in ("TreeEnsembleRegressor", "TreeEnsembleClassifier")
    is_classifier = op_type == "TreeEnsembleClassifier"

    base_values = attrs.get("base_values", {"floats": [0.0]})["floats"]
    assert len(base_values) == 1, "Only one base value is supported"
    post = attrs.get("post_transform", {"s": b"NONE"})["s"].decode()
    transform = {"NONE": IDENTITY, "SOFTMAX": SOFTMAX, "LOGISTIC": SIGMOID}[post]
    if "nodes_missing_value_tracks_true" in attrs:
        assert not any(attrs["nodes_missing_value_tracks_true"]["ints"])
    modes = [m.decode() for m in attrs["nodes_modes"]["strings"]]
    cmp_modes = {m for m in modes[1:] if m != "LEAF"}       # scan starts at 1 (:131)
    assert len(cmp_modes) == 1, "Only one node mode is supported"
    predicate = {"BRANCH_LT": PRED_LT, "BRANCH_GEQ": PRED_GE,
                 "BRANCH_GT": PRED_GT, "BRANCH_LEQ": PRED_LE}[cmp_modes.pop()]
    tree_ids = attrs["nodes_treeids"]["ints"]
    node_ids = attrs["nodes_nodeids"]["ints"]
    feat = attrs["nodes_featureids"]["ints"]
    vals = attrs["nodes_values"]["floats"]
    true_ids = attrs["nodes_truenodeids"]["ints"]
    false_ids = attrs["nodes_falsenodeids"]["ints"]
    num_nodes = len(node_ids)
    n_classes = (attrs.get("n_targets", {"i": 0})["i"] or 0) if is_classifier else 0

    value = {}
    for i in range(num_nodes):
        value[(tree_ids[i], node_ids[i])] = [feat[i], float(np.float32(vals[i])), None, None]
    for i in range(num_nodes):
        key = (tree_ids[i], node_ids[i])
        for slot, ids in ((2, true_ids), (3, false_ids)):       # true = left (:227-228)
            ck = (tree_ids[i], ids[i])
            assert ck in value, "child not found"
            if 0 < ids[i] < num_nodes:
                value[key][slot] = ck
    roots, cur = [], None
    for i in range(num_nodes):
        if cur is None or tree_ids[i] != cur:
            roots.append((tree_ids[i], node_ids[i]))
        cur = tree_ids[i]
    tree_classes = {}
    t_tree, t_node = attrs["target_treeids"]["ints"], attrs["target_nodeids"]["ints"]
    t_ids, t_w = attrs["target_ids"]["ints"], attrs["target_weights"]["floats"]
    for i in range(len(t_w)):
        key = (t_tree[i], t_node[i])
        assert key in value, "Key not found"
        tree_classes.setdefault(t_tree[i], set()).add(t_ids[i])
        value[key][1] = float(np.float32(t_w[i]))

    trees, class_ids = [], []
    for idx, root in enumerate(roots):
        thr, fi, le, ri = [], [], [], []
        # pre-order numbering: node, then left subtree, then right subtree (:315-334)
        stack = [(root, -1, 0)]
        while stack:
            key, parent, side = stack.pop()
            me = len(thr)
            f_, v_, l_, r_ = value[key]
            thr.append(v_); fi.append(f_); le.append(-1); ri.append(-1)
            if parent >= 0:
                (le if side == 0 else ri)[parent] = me
            if r_ is not None:
                stack.append((r_, me, 1))
            if l_ is not None:
                stack.append((l_, me, 0))
        trees.append((thr, fi, le, ri))
        if is_classifier and n_classes > 0:
            cls = tree_classes.get(idx, set())
            assert len(cls) == 1
            class_ids.append(next(iter(cls)))
        else:
            class_ids.append(0)
    return _assemble(trees, num_features=num_features, initial_value=float(np.float32(base_values[0])),
                     transform=transform, num_classes=int(n_classes), predicate=predicate,
                     class_id=np.asarray(class_ids, dtype=np.int32), meta={"op_type": op_type})


def read_csv(path, max_rows=None):
    """Golden CSVs: no header, F feature columns then one expected value
    (src/test/TestUtilsCommon.cpp:16-56)."""
    with _open_text(path) as fh:
        data = np.loadtxt(fh, delimiter=",", dtype=np.float64, max_rows=max_rows, ndmin=2)
    return data[:, :-1], data[:, -1]

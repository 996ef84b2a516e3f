"""Writes a TreeEnsembleRegressor / TreeEnsembleClassifier ONNX file from flat
tree arrays (protobuf wire format by hand; field numbers as in onnx.proto).
Test helper: lets the suite produce models in every comparison mode."""
import struct


def _varint(v):
    if v < 0:
        v += 1 << 64
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _key(field, wt):
    return _varint((field << 3) | wt)


def _bytes_field(field, payload):
    return _key(field, 2) + _varint(len(payload)) + payload


def _attr(name, ints=None, floats=None, strings=None, s=None, i=None, packed=False):
    body = _bytes_field(1, name.encode())
    if i is not None:
        body += _key(3, 0) + _varint(i)
    if s is not None:
        body += _bytes_field(4, s.encode())
    if floats is not None:
        if packed:
            body += _bytes_field(7, b"".join(struct.pack("<f", f) for f in floats))
        else:
            body += b"".join(_key(7, 5) + struct.pack("<f", f) for f in floats)
    if ints is not None:
        if packed:
            body += _bytes_field(8, b"".join(_varint(v) for v in ints))
        else:
            body += b"".join(_key(8, 0) + _varint(v) for v in ints)
    if strings is not None:
        body += b"".join(_bytes_field(9, t.encode()) for t in strings)
    return _bytes_field(5, body)


def write_onnx(path, trees, mode="BRANCH_LT", base_value=0.0, post_transform="NONE", classifier=False,
               n_classes=0, class_ids=None, packed=False):
    """trees: list of (value, feature, left, right) with local child indices (-1 on leaves); node ids
    are the local indices, the true branch is `left`.  class_ids[t] is the class tree t votes for, or a
    sequence that gives every leaf of tree t (in node order) a class id of its own."""
    tree_ids, node_ids, feats, vals, true_ids, false_ids, modes = [], [], [], [], [], [], []
    t_tree, t_node, t_ids, t_w = [], [], [], []
    for t, (value, feature, left, right) in enumerate(trees):
        for n in range(len(value)):
            leaf = left[n] == -1
            tree_ids.append(t); node_ids.append(n)
            feats.append(0 if leaf else int(feature[n]))
            vals.append(0.0 if leaf else float(value[n]))
            true_ids.append(0 if leaf else int(left[n]))
            false_ids.append(0 if leaf else int(right[n]))
            modes.append("LEAF" if leaf else mode)
            if leaf:
                cls = class_ids[t] if class_ids is not None else 0
                if hasattr(cls, "__len__"):
                    cls = cls[len([m for m in t_tree if m == t]) % len(cls)]
                t_tree.append(t); t_node.append(n)
                t_ids.append(int(cls))
                t_w.append(float(value[n]))
    node = _bytes_field(4, b"TreeEnsembleClassifier" if classifier else b"TreeEnsembleRegressor")
    node += _attr("base_values", floats=[base_value], packed=packed)
    node += _attr("n_targets", i=n_classes if classifier else 1)
    node += _attr("nodes_falsenodeids", ints=false_ids, packed=packed)
    node += _attr("nodes_featureids", ints=feats, packed=packed)
    node += _attr("nodes_missing_value_tracks_true", ints=[0] * len(node_ids), packed=packed)
    node += _attr("nodes_modes", strings=modes)
    node += _attr("nodes_nodeids", ints=node_ids, packed=packed)
    node += _attr("nodes_treeids", ints=tree_ids, packed=packed)
    node += _attr("nodes_truenodeids", ints=true_ids, packed=packed)
    node += _attr("nodes_values", floats=vals, packed=packed)
    node += _attr("post_transform", s=post_transform)
    node += _attr("target_ids", ints=t_ids, packed=packed)
    node += _attr("target_nodeids", ints=t_node, packed=packed)
    node += _attr("target_treeids", ints=t_tree, packed=packed)
    node += _attr("target_weights", floats=t_w, packed=packed)
    node += _bytes_field(7, b"ai.onnx.ml")
    graph = _bytes_field(1, node)
    model = _key(1, 0) + _varint(7) + _bytes_field(7, graph)
    with open(path, "wb") as fh:
        fh.write(model)

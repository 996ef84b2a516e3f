"""Host-side logic of the runtime library, runnable without a GPU: the C-ABI
exports everything include/tbruntime_amd.h declares, the C++ loaders build the
same forests as the oracle's loaders, packing round-trips, and errors come
back as messages instead of aborts (the reference asserts,
src/json/xgboostparser.h:100, src/runtime/runtime.cpp:172)."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

from oracle import model_io
from treebeard_amd import runtime_api, synth

from conftest import BENCHMARK_XGB, GOLDEN, ROOT, benchmark_model, random_models
from onnx_writer import write_onnx


@pytest.fixture(scope="module")
def lib():
    return runtime_api.api().runtime_lib


def last_error():
    return runtime_api.api().last_error()


def load_forest(lib, path, kind="xgboost_json", num_features=0):
    h = lib.tbmi_load_forest(str(path).encode(), kind.encode(), num_features)
    assert h, last_error()
    return h


def forest_arrays(lib, h):
    info = (ctypes.c_int64 * 6)()
    init = ctypes.c_double()
    assert lib.tbmi_forest_info(h, info, ctypes.byref(init)) == 0
    trees = []
    for t in range(info[0]):
        n = lib.tbmi_forest_tree_size(h, t)
        v, f = np.empty(n, np.float32), np.empty(n, np.int32)
        l, r = np.empty(n, np.int32), np.empty(n, np.int32)
        c = ctypes.c_int32()
        assert lib.tbmi_forest_tree(h, t, v.ctypes.data, f.ctypes.data, l.ctypes.data, r.ctypes.data, ctypes.byref(c)) == 0
        trees.append((v, f, l, r, c.value))
    return list(info), init.value, trees


def assert_same_forest(lib, h, forest):
    info, init, trees = forest_arrays(lib, h)
    assert info[:5] == [forest.num_trees, forest.num_features, forest.num_classes, forest.transform, forest.predicate]
    assert info[5] == len(forest.threshold)
    assert init == forest.initial_value
    for t, (v, f, l, r, c) in enumerate(trees):
        thr, feat, left, right = forest.tree(t)
        np.testing.assert_array_equal(v.astype(np.float64), thr)
        np.testing.assert_array_equal(l, left)
        np.testing.assert_array_equal(r, right)
        internal = left != -1
        np.testing.assert_array_equal(f[internal], feat[internal])
        assert c == forest.class_id[t]


def test_every_declared_symbol_is_exported(lib):
    header = open(os.path.join(ROOT, "include", "tbruntime_amd.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    header = header.replace("#define TBAMD_EXPORT", "")
    names = re.findall(r"TBAMD_EXPORT\s+[^;(]*?\b(\w+)\s*\(", header)
    assert len(names) > 70
    for name in names:
        assert hasattr(lib, name), name
    assert set(runtime_api.SIGNATURES) == set(names)


@pytest.mark.parametrize("path", random_models()[::2] + [benchmark_model(n) for n in BENCHMARK_XGB], ids=os.path.basename)
def test_xgboost_loader_matches_oracle_loader(lib, plain_file, path):
    h = load_forest(lib, plain_file(path))
    assert_same_forest(lib, h, model_io.load_xgboost_json(path))
    lib.tbmi_delete_forest(h)


@pytest.mark.parametrize("k", [1, 2, 3, 5])
def test_synthetic_models_load_and_pack(lib, synth_model, k):
    path = synth_model(k)
    h = load_forest(lib, path)
    assert_same_forest(lib, h, model_io.load_xgboost_json(path))
    stats = (ctypes.c_int64 * 5)()
    for rows_per_block, interleave, group_bytes in [(256, 4, 49152), (128, 8, 32768), (64, 1, 16384), (256, 2, 16384)]:
        assert lib.tbmi_pack_roundtrip(h, rows_per_block, interleave, group_bytes, stats) == 0, last_error()
        assert stats[3] <= 160 * 1024
    lib.tbmi_delete_forest(h)


def test_onnx_loader_matches_oracle_loader(lib, plain_file):
    path = os.path.join(GOLDEN, "benchmark", "abalone_onnx_model_save.onnx.gz")
    h = load_forest(lib, plain_file(path), "onnx_file", 8)
    assert_same_forest(lib, h, model_io.load_onnx(path, 8))
    lib.tbmi_delete_forest(h)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("mode", ["BRANCH_LT", "BRANCH_GEQ", "BRANCH_GT", "BRANCH_LEQ"])
def test_onnx_comparison_modes_and_encodings(lib, tmp_path, mode, packed):
    rng = np.random.default_rng(3)
    trees = [(rng.normal(size=7).astype(np.float32), rng.integers(0, 4, 7), [1, 3, 5, -1, -1, -1, -1], [2, 4, 6, -1, -1, -1, -1])
             for _ in range(5)]
    path = tmp_path / "m.onnx"
    write_onnx(path, trees, mode=mode, base_value=0.25, packed=packed)
    forest = model_io.load_onnx(path, 4)
    assert forest.predicate == ["BRANCH_LT", "BRANCH_GEQ", "BRANCH_GT", "BRANCH_LEQ"].index(mode)
    h = load_forest(lib, path, "onnx_file", 4)
    assert_same_forest(lib, h, forest)
    stats = (ctypes.c_int64 * 5)()
    assert lib.tbmi_pack_roundtrip(h, 64, 2, 4096, stats) == 0, last_error()
    lib.tbmi_delete_forest(h)


def preorder_trees(rng, count, num_features, max_depth=5):
    """Random trees numbered in pre-order (node, left subtree, right subtree) - the numbering both ONNX loaders
    give their nodes (src/json/onnxmodelparser.h:315-334) - so that a loaded tree can be compared with what
    the writer was handed index by index."""
    trees = []
    for _ in range(count):
        value, feature, left, right = [], [], [], []

        def grow(depth):
            me = len(value)
            value.append(0.0); feature.append(0); left.append(-1); right.append(-1)
            if depth < max_depth and (depth == 0 or rng.random() < 0.7):
                value[me] = float(np.float32(rng.normal()))
                feature[me] = int(rng.integers(0, num_features))
                left[me] = grow(depth + 1)
                right[me] = grow(depth + 1)
            else:
                value[me] = float(np.float32(rng.normal(0.0, 0.3)))
            return me

        grow(0)
        trees.append((np.asarray(value, np.float32), np.asarray(feature, np.int32), left, right))
    return trees


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("post_transform,transform", [("NONE", model_io.IDENTITY), ("LOGISTIC", model_io.SIGMOID),
                                                      ("SOFTMAX", model_io.SOFTMAX)])
def test_onnx_classifier_comes_back_as_written(lib, tmp_path, post_transform, transform, packed):
    """TreeEnsembleClassifier (src/json/onnxmodelparser.h:102-113 post_transform, :162-172 n_targets only counts
    for classifiers, :355-374 one class id per tree): the forest handed to the writer - thresholds, features,
    links, leaf weights, class id per tree, base value, transform - comes back field for field from the C++
    loader and from the oracle's loader, and the oracle's class ids on that forest are those of the reference's
    own DecisionForest::Predict_Float fed the same arrays through NewTree/NewNode."""
    from oracle import cpu_oracle
    rng = np.random.Generator(np.random.PCG64(31 + len(post_transform)))
    classes, features = 5, 6
    trees = preorder_trees(rng, 23, features)
    class_ids = [int(c) for c in rng.integers(0, classes, len(trees))]
    path = tmp_path / "classifier.onnx"
    write_onnx(path, trees, base_value=0.125, post_transform=post_transform, classifier=True, n_classes=classes,
               class_ids=class_ids, packed=packed)
    written = model_io._assemble([(t[0].astype(np.float64), t[1], t[2], t[3]) for t in trees], num_features=features,
                                 initial_value=0.125, transform=transform, num_classes=classes, predicate=model_io.PRED_LT,
                                 class_id=np.asarray(class_ids, np.int32), meta={})
    loaded = model_io.load_onnx(path, features)
    assert (loaded.num_trees, loaded.num_features, loaded.num_classes, loaded.transform, loaded.predicate,
            loaded.initial_value) == (len(trees), features, classes, transform, model_io.PRED_LT, 0.125)
    np.testing.assert_array_equal(loaded.class_id, class_ids)
    for t in range(len(trees)):
        for got, want in zip(loaded.tree(t), written.tree(t)):          # thresholds / leaf weights, features, left, right
            np.testing.assert_array_equal(got, want)
    h = load_forest(lib, path, "onnx_file", features)
    assert_same_forest(lib, h, written)
    lib.tbmi_delete_forest(h)
    # a regressor with the same attributes has no classes (n_targets is looked at for classifiers only)
    write_onnx(tmp_path / "regressor.onnx", trees, base_value=0.125, post_transform="NONE", classifier=False, n_classes=classes,
               class_ids=class_ids, packed=packed)
    assert model_io.load_onnx(tmp_path / "regressor.onnx", features).num_classes == 0
    h = load_forest(lib, tmp_path / "regressor.onnx", "onnx_file", features)
    info, _, _ = forest_arrays(lib, h)
    assert info[2] == 0
    lib.tbmi_delete_forest(h)
    # class ids of the oracle on the loaded forest = the reference's own walk + per-class sums + arg-max
    x = rng.normal(size=(500, features)).astype(np.float32)
    pred, sums = cpu_oracle.predict(loaded, x)
    top2 = np.sort(sums, axis=1)[:, -2:]
    assert (top2[:, 1] > top2[:, 0]).all()            # no exact ties: the two tie rules do not come into play
    np.testing.assert_array_equal(pred, np.argmax(sums, axis=1))
    if cpu_oracle.ref_available():
        as_softmax = model_io._assemble([(t[0].astype(np.float64), t[1], t[2], t[3]) for t in trees], num_features=features,
                                        initial_value=0.125, transform=model_io.SOFTMAX, num_classes=classes,
                                        predicate=model_io.PRED_LT, class_id=np.asarray(class_ids, np.int32), meta={})
        ref = cpu_oracle.RefForest(as_softmax)        # (Predict_Float insists on the soft-max transform for classifiers)
        np.testing.assert_array_equal(ref.predict_float(x), pred.astype(np.float32))
        np.testing.assert_array_equal(ref.predict_double(x.astype(np.float64)), pred.astype(np.float64))


def test_onnx_classifier_with_several_class_ids_in_one_tree_is_refused(lib, tmp_path):
    """src/json/onnxmodelparser.h:364-367 asserts one class id per tree; here the loaders say so."""
    rng = np.random.Generator(np.random.PCG64(5))
    trees = preorder_trees(rng, 4, 3)
    path = tmp_path / "mixed.onnx"
    write_onnx(path, trees, classifier=True, n_classes=3, class_ids=[0, 1, [0, 2], 1])
    assert lib.tbmi_load_forest(str(path).encode(), b"onnx_file", 3) == 0
    assert "multiple class IDs per tree" in last_error()
    with pytest.raises(AssertionError):
        model_io.load_onnx(path, 3)
    write_onnx(path, trees, classifier=False, n_classes=3, class_ids=[0, 1, [0, 2], 1])       # regressors do not look
    assert model_io.load_onnx(path, 3).num_classes == 0
    h = load_forest(lib, path, "onnx_file", 3)
    lib.tbmi_delete_forest(h)


def test_global_layout_round_trips(lib, synth_model):
    for k in (1, 3, 5):
        h = load_forest(lib, synth_model(k))
        stats = (ctypes.c_int64 * 5)()
        assert lib.tbmi_pack_roundtrip(h, 256, 4, 0, stats) == 0, last_error()
        forest = model_io.load_xgboost_json(synth_model(k))
        assert stats[0] == 0 and stats[2] == len(forest.threshold) and stats[3] == 0
        lib.tbmi_delete_forest(h)


def test_pack_rejects_plans_that_cannot_hold_the_model(lib, synth_model):
    h = load_forest(lib, synth_model(5))
    stats = (ctypes.c_int64 * 5)()
    assert lib.tbmi_pack_roundtrip(h, 256, 4, 2048, stats) == -1      # deepest tree > one group
    assert "does not fit" in last_error()
    assert lib.tbmi_pack_roundtrip(h, 256, 3, 65536, stats) == -1     # interleave not a power of two
    assert lib.tbmi_pack_roundtrip(h, 1024, 4, 65536, stats) == -1    # 16-bit feature offsets overflow
    assert "16 bits" in last_error()
    lib.tbmi_delete_forest(h)


def test_loader_errors_are_reported_not_fatal(lib, tmp_path):
    assert lib.tbmi_load_forest(b"/nonexistent/model.json", b"xgboost_json", 0) == 0
    assert "cannot open" in last_error()
    bad = tmp_path / "bad.json"
    bad.write_text("{\"learner\": ")
    assert lib.tbmi_load_forest(str(bad).encode(), b"xgboost_json", 0) == 0
    assert "JSON" in last_error()
    # unknown objective (the reference asserts: src/json/xgboostparser.h:94-102)
    rng = np.random.Generator(np.random.PCG64(1))
    tree = synth._grow_tree(rng, 2, lambda d, s: 1.0, lambda: (0, 0.5), lambda: 1.0)
    path = tmp_path / "obj.json"
    synth.write_xgboost_json(path, [tree], 2, objective="rank:pairwise")
    assert lib.tbmi_load_forest(str(path).encode(), b"xgboost_json", 0) == 0
    assert "Unknown objective" in last_error()
    # feature index outside the declared features
    doc = json.load(open(path))
    doc["learner"]["objective"]["name"] = "reg:squarederror"
    doc["learner"]["gradient_booster"]["model"]["trees"][0]["split_indices"][0] = 9
    path.write_text(json.dumps(doc))
    assert lib.tbmi_load_forest(str(path).encode(), b"xgboost_json", 0) == 0
    assert "feature index" in last_error()
    assert lib.tbmi_load_forest(str(path).encode(), b"treelite", 0) == 0
    assert "unknown forest creator" in last_error()
    # ONNX needs the feature count from the options (src/json/onnxmodelparser.h:345-348)
    assert lib.tbmi_load_forest(os.path.join(GOLDEN, "handbuilt", "x.onnx").encode(), b"onnx_file", 0) == 0
    assert "Number of features" in last_error()


def test_option_handles_and_switches(lib):
    o = lib.CreateCompilerOptions()
    for name in runtime_api.OPTION_SETTERS:
        getattr(lib, "Set_" + name)(o, 1)
    lib.Set_tilingType(o, 7)
    assert "Invalid tiling type" in last_error()
    lib.Set_statsProfileCSVPath(o, b"/tmp/profile.csv")
    lib.DeleteCompilerOptions(o)
    g = lib.CreateGPUAutoScheduleOptions()
    for name in runtime_api.GPU_OPTION_SETTERS:
        getattr(lib, "Set_" + name)(g, 2)
    lib.DeleteGPUAutoScheduleOptions(g)
    lib.SetEnableSparseRepresentation(1)
    assert lib.IsSparseRepresentationEnabled() == 1
    lib.SetEnableSparseRepresentation(0)
    lib.SetPeeledCodeGenForProbabilityBasedTiling(1)
    assert lib.IsPeeledCodeGenForProbabilityBasedTilingEnabled() == 1
    lib.SetPeeledCodeGenForProbabilityBasedTiling(0)
    assert lib.GetBatchSize(0) == -1 and "null" in last_error()


def test_synthetic_configurations_have_the_stated_shape(synth_model):
    f1 = model_io.load_xgboost_json(synth_model(1))
    assert (f1.num_trees, f1.num_features, f1.transform, f1.initial_value) == (100, 8, model_io.IDENTITY, 0.5)
    assert all(f1.depth(t) == 6 and len(f1.tree(t)[0]) == 127 for t in range(100))
    f2 = model_io.load_xgboost_json(synth_model(2))
    assert (f2.num_trees, f2.num_features, f2.transform, f2.initial_value) == (1000, 28, model_io.SIGMOID, 0.0)
    assert max(f2.depth(t) for t in range(1000)) == 8
    f3 = model_io.load_xgboost_json(synth_model(3))
    assert (f3.num_trees, f3.num_features, f3.num_classes) == (800, 54, 8)
    np.testing.assert_array_equal(f3.class_id, np.arange(800) % 8)
    f5 = model_io.load_xgboost_json(synth_model(5))
    assert (f5.num_trees, f5.num_features) == (800, 90) and max(f5.depth(t) for t in range(800)) == 12
    x3 = synth.CONFIGS[3].batch_rows(2000)
    assert set(np.unique(x3[:, 10:])) <= {0.0, 1.0} and 0.05 < x3[:, 10:].mean() < 0.15


def test_hit_count_profile_of_the_reference_matches_its_model(lib, plain_file):
    """xgb_models/profiles/higgs.test.csv against higgs_xgb_model_save.json: per tree the leaf hits add up to numRows."""
    h = load_forest(lib, plain_file(benchmark_model("higgs")))
    rows, steps = ctypes.c_int64(), ctypes.c_double()
    profile = plain_file(os.path.join(GOLDEN, "benchmark", "higgs.test.profile.csv.gz"))
    assert lib.tbmi_forest_load_profile(h, profile.encode(), ctypes.byref(rows), ctypes.byref(steps)) == 0, last_error()
    assert rows.value > 1000 and 100 * 1.0 < steps.value <= 100 * 8.0     # 100 trees, depth <= 8
    lib.tbmi_delete_forest(h)
    # a profile of another model is refused
    h = load_forest(lib, plain_file(benchmark_model("airline")))
    assert lib.tbmi_forest_load_profile(h, profile.encode(), ctypes.byref(rows), ctypes.byref(steps)) == -1
    assert "hit-count profile" in last_error()
    lib.tbmi_delete_forest(h)


def test_hit_count_profile_agrees_with_oracle_walks(lib, tmp_path, synth_model):
    """A profile written from the oracle's leaf ids in the reference's format reads back with the oracle's step count."""
    from oracle import cpu_oracle
    forest = model_io.load_xgboost_json(synth_model(1))
    x = synth.CONFIGS[1].batch_rows(500)
    ids, plen = cpu_oracle.leaf_ids(forest, x, want_path_len=True)
    lines = ["%d, %d" % (forest.num_trees, x.shape[0])]
    for t in range(forest.num_trees):
        _, _, left, _ = forest.tree(t)
        leaves = np.nonzero(left == -1)[0]
        hits = [(int((ids[:, t] == leaf).sum()), 6) for leaf in leaves]
        lines.append(", ".join("%d, %d" % hd for hd in hits))
    path = tmp_path / "profile.csv"
    path.write_text("\n".join(lines) + "\n")
    h = load_forest(lib, synth_model(1))
    rows, steps = ctypes.c_int64(), ctypes.c_double()
    assert lib.tbmi_forest_load_profile(h, str(path).encode(), ctypes.byref(rows), ctypes.byref(steps)) == 0, last_error()
    assert rows.value == 500 and abs(steps.value - plen.sum() / 500) < 1e-9
    lib.tbmi_delete_forest(h)


def test_c_client_builds_against_the_header_and_sees_documented_errors(tmp_path, synth_model):
    """The public header is plain C; a C99 program links the library and meets the documented error behaviour
    (0 / -1 and a message, never an abort; no CPU fallback when there is no device)."""
    import shutil
    import subprocess
    from treebeard_amd.runtime_api import LIB_PATH
    if shutil.which("gcc") is None:
        pytest.skip("needs gcc")
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
    exe = str(tmp_path / "abi_client")
    libdir = os.path.dirname(LIB_PATH)
    build = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(root, "include"),
                            os.path.join(root, "tests", "native", "abi_client.c"), "-L", libdir, "-ltreebeard_amd",
                            "-Wl,-rpath," + libdir, "-o", exe], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe, synth_model(1)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)
    assert "trees=100 features=8 classes=0" in run.stdout

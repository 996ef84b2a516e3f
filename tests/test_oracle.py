"""Pins the CPU oracle (oracle/) before anything is compared against it.

  * the XGBoost / ONNX-runtime golden CSVs the reference ships with its models
    (last column = the library's own prediction, src/test/TestUtilsCommon.h:156-216)
  * the reference's own scalar walker compiled from its header (oracle/_ref), when built
  * brute-force python walks, closed forms (expit, softmax), explicit tie cases
  * the hand-built trees whose expected dense arrays are literal in
    src/test/ForestTestUtils.h:78-79, :118-119
"""
import os

import numpy as np
import pytest
import scipy.special

from oracle import cpu_oracle, model_io
from treebeard_amd import synth

from conftest import BENCHMARK_XGB, GOLDEN, benchmark_csv, benchmark_model, random_models

needs_ref = pytest.mark.skipif(not cpu_oracle.ref_available(), reason="oracle/_ref not built (no reference checkout)")


def brute_force_leaf(forest, t, row):
    thr, feat, left, right = forest.tree(t)
    n = 0
    while left[n] != -1:
        n = left[n] if np.float32(row[feat[n]]) < np.float32(thr[n]) else right[n]
    return n


@pytest.mark.parametrize("path", random_models(), ids=os.path.basename)
def test_random_models_match_xgboost_csv(path):
    forest = model_io.load_xgboost_json(path)
    x, expected = model_io.read_csv(path + ".csv")
    pred, _ = cpu_oracle.predict(forest, x.astype(np.float32))
    # XGBoost accumulates in f32; the oracle (like the reference's) in double
    np.testing.assert_allclose(pred, expected, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("name", BENCHMARK_XGB)
def test_benchmark_models_match_xgboost_csv(name):
    forest = model_io.load_xgboost_json(benchmark_model(name))
    x, expected = model_io.read_csv(benchmark_csv(name))
    pred, _ = cpu_oracle.predict(forest, x.astype(np.float32))
    if forest.transform == model_io.SIGMOID:
        np.testing.assert_allclose(pred, expected, rtol=0, atol=1e-6)
    else:
        np.testing.assert_allclose(pred, expected, rtol=1e-5, atol=0)


def test_onnx_abalone_matches_onnxruntime_csv():
    forest = model_io.load_onnx(os.path.join(GOLDEN, "benchmark", "abalone_onnx_model_save.onnx.gz"), 8)
    assert forest.num_trees == 1000 and forest.predicate == model_io.PRED_LT
    x, expected = model_io.read_csv(os.path.join(GOLDEN, "benchmark", "abalone_onnx_model_save.onnx.csv"))
    pred, _ = cpu_oracle.predict(forest, x.astype(np.float32))
    np.testing.assert_allclose(pred, expected, rtol=1e-5, atol=0)


def test_onnx_and_json_give_the_same_forest():
    fo = model_io.load_onnx(os.path.join(GOLDEN, "benchmark", "higgs_xgb_model_save.onnx.gz"), 28)
    fx = model_io.load_xgboost_json(benchmark_model("higgs"))
    assert fo.num_trees == fx.num_trees and len(fo.threshold) == len(fx.threshold)
    x, _ = model_io.read_csv(benchmark_csv("higgs"))
    x = x.astype(np.float32)
    # node numbering differs (pre-order vs XGBoost ids): compare leaf VALUES reached
    vo = fo.threshold[(fo.tree_offsets[:-1][None, :] + cpu_oracle.leaf_ids(fo, x))]
    vx = fx.threshold[(fx.tree_offsets[:-1][None, :] + cpu_oracle.leaf_ids(fx, x))]
    np.testing.assert_array_equal(vo, vx)


@needs_ref
@pytest.mark.parametrize("path", random_models()[::3] + [benchmark_model(n) for n in BENCHMARK_XGB], ids=os.path.basename)
def test_oracle_equals_reference_header(path):
    forest = model_io.load_xgboost_json(path)
    csv = path[:-3] + ".csv" if path.endswith(".gz") else path + ".csv"
    x, _ = model_io.read_csv(csv)
    x32 = x.astype(np.float32)
    ref = cpu_oracle.RefForest(forest)
    pred, _ = cpu_oracle.predict(forest, x32)
    np.testing.assert_array_equal(pred, ref.predict_float(x32))                       # Predict_Float
    np.testing.assert_array_equal(cpu_oracle.predict_f64(forest, x), ref.predict_double(x))  # Predict
    ids = cpu_oracle.leaf_ids(forest, x32)
    values = forest.threshold[forest.tree_offsets[:-1][None, :] + ids].astype(np.float32)
    np.testing.assert_array_equal(values, ref.tree_values_float(x32))                 # PredictTree_Float


@needs_ref
def test_multiclass_equals_reference_header():
    rng = np.random.default_rng(5)
    trees = []
    for t in range(12):
        thr = rng.normal(size=7).astype(np.float32)
        trees.append((thr, rng.integers(0, 5, 7), [1, 3, 5, -1, -1, -1, -1], [2, 4, 6, -1, -1, -1, -1]))
    forest = model_io._assemble(trees, num_features=5, initial_value=0.5, transform=model_io.SOFTMAX, num_classes=4,
                                predicate=model_io.PRED_LT, class_id=np.arange(12, dtype=np.int32) % 4)
    x = rng.normal(size=(500, 5)).astype(np.float32)
    pred, sums = cpu_oracle.predict(forest, x)
    np.testing.assert_array_equal(pred, cpu_oracle.RefForest(forest).predict_float(x))
    np.testing.assert_array_equal(pred, np.argmax(sums.astype(np.float32), axis=1))


def test_leaf_ids_match_brute_force():
    forest = model_io.load_xgboost_json(os.path.join(GOLDEN, "Random_4Tree", sorted(os.listdir(os.path.join(GOLDEN, "Random_4Tree")))[0]))
    rng = np.random.default_rng(1)
    x = rng.uniform(-10, 10, size=(64, forest.num_features)).astype(np.float32)
    ids, plen = cpu_oracle.leaf_ids(forest, x, want_path_len=True)
    for r in range(x.shape[0]):
        for t in range(forest.num_trees):
            assert ids[r, t] == brute_force_leaf(forest, t, x[r])
    assert cpu_oracle.total_steps(forest, x) == int(plen.sum())


def test_threshold_equal_goes_right():
    # x == threshold is "not less": right child (src/include/DecisionForest.h:372-375)
    forest = model_io._assemble([([0.5, 1.0, 2.0], [0, 0, 0], [1, -1, -1], [2, -1, -1])], num_features=1,
                                initial_value=0.0, transform=model_io.IDENTITY, num_classes=0,
                                predicate=model_io.PRED_LT, class_id=np.zeros(1, np.int32))
    x = np.array([[0.5], [np.nextafter(np.float32(0.5), np.float32(0))], [np.nan]], dtype=np.float32)
    pred, _ = cpu_oracle.predict(forest, x)
    np.testing.assert_array_equal(pred, [2.0, 1.0, 2.0])   # NaN compares false: right


def dense_arrays(forest, t):
    """DecisionForest.h:292-315 restated for the test: 2^depth-1 slots, holes (0, -1)."""
    thr, feat, left, right = forest.tree(t)
    depth = forest.depth(t) + 1
    out_thr, out_idx = np.zeros(2 ** depth - 1), np.full(2 ** depth - 1, -1)

    def fill(slot, n):
        out_thr[slot] = thr[n]
        out_idx[slot] = -1 if left[n] == -1 else feat[n]
        if left[n] != -1:
            fill(2 * slot + 1, left[n])
            fill(2 * slot + 2, right[n])
    fill(0, 0)
    return out_thr, out_idx


HANDBUILT = {
    "leftheavy": ([0.5, 0.3, 0.8, 0.1, 0.2, 0, 0], [2, 4, -1, -1, -1, -1, -1]),
    "rightheavy": ([0.5, 0.85, 0.3, 0, 0, 0.15, 0.25], [2, -1, 4, -1, -1, -1, -1]),
}


@pytest.mark.parametrize("name", sorted(HANDBUILT))
def test_handbuilt_trees_expected_arrays(name):
    forest = model_io.load_xgboost_json(os.path.join(GOLDEN, "handbuilt", name + "_xgb_model.json"), threshold_f32=False)
    thr, idx = dense_arrays(forest, 0)
    np.testing.assert_array_equal(thr, HANDBUILT[name][0])
    np.testing.assert_array_equal(idx, HANDBUILT[name][1])
    if cpu_oracle.ref_available():
        rthr, ridx = cpu_oracle.RefForest(forest).dense_arrays(0)
        np.testing.assert_array_equal(rthr, thr)
        np.testing.assert_array_equal(ridx, idx)


def test_sigmoid_closed_form():
    forest = model_io._assemble([([0.0, -3.0, 2.5], [0, 0, 0], [1, -1, -1], [2, -1, -1])], num_features=1,
                                initial_value=0.25, transform=model_io.SIGMOID, num_classes=0,
                                predicate=model_io.PRED_LT, class_id=np.zeros(1, np.int32))
    pred, sums = cpu_oracle.predict(forest, np.array([[-1.0], [1.0]], dtype=np.float32))
    np.testing.assert_array_equal(sums, [-2.75, 2.75])
    np.testing.assert_allclose(pred, scipy.special.expit(np.array([-2.75, 2.75])).astype(np.float32), rtol=0, atol=6e-8)


def test_argmax_tie_rules_and_softmax():
    sums = np.array([[1.0, 3.0, 3.0, 2.0], [5.0, 5.0, 5.0, 5.0], [-1.0, -2.0, -0.5, -0.5]], dtype=np.float32)
    # generated code: ties go to the larger class id (src/mlir/LowerReduceOps.cpp:148-187)
    np.testing.assert_array_equal(cpu_oracle.argmax_generated(sums), [2, 3, 3])
    # reference oracle: std::max_element, first maximum (src/include/DecisionForest.h:446-468)
    np.testing.assert_array_equal(np.argmax(sums, axis=1), [1, 0, 2])
    np.testing.assert_allclose(cpu_oracle.softmax(sums.astype(np.float64)), scipy.special.softmax(sums.astype(np.float64), axis=1),
                               rtol=1e-14)


def test_tree_outer_schedule_matches_default_within_f32():
    forest = model_io.load_xgboost_json(benchmark_model("higgs"))
    x, _ = model_io.read_csv(benchmark_csv("higgs"))
    x = x.astype(np.float32)
    pred, _ = cpu_oracle.predict(forest, x)
    order = np.argsort([forest.depth(t) for t in range(forest.num_trees)], kind="stable").astype(np.int32)
    out = cpu_oracle.predict_tree_outer(forest, x, tree_order=order, threads=3)
    np.testing.assert_allclose(out, pred, rtol=0, atol=1e-6)


# --------------------------------------------------------------------------
# tiled CPU walk (the reference's vectorised CPU path, oracle/tiled_oracle.c)
# --------------------------------------------------------------------------
@pytest.mark.parametrize("tile_size", [1, 2, 3, 4, 8])
def test_tiled_walk_reaches_the_scalar_leaf_on_reference_models(tile_size):
    paths = random_models()[::4] + [benchmark_model("higgs"), benchmark_model("year_prediction_msd")]
    for path in paths:
        forest = model_io.load_xgboost_json(path)
        csv = path[:-3] + ".csv" if path.endswith(".gz") else path + ".csv"
        x, _ = model_io.read_csv(csv, max_rows=120)
        x = x.astype(np.float32)
        tiled = cpu_oracle.TiledForest(forest, tile_size)
        np.testing.assert_array_equal(tiled.leaf_ids(x), cpu_oracle.leaf_ids(forest, x))


@pytest.mark.parametrize("tile_size", [2, 3, 4, 8])
def test_tiled_walk_on_random_and_degenerate_trees(tile_size, tmp_path):
    from treebeard_amd import synth
    rng = np.random.Generator(np.random.PCG64(tile_size))
    trees = [synth._grow_tree(rng, 9, lambda d, s: 0.75, lambda: (rng.integers(0, 6), np.round(rng.normal(), 1)),
                              lambda: rng.normal()) for _ in range(60)]
    trees.append(synth._grow_tree(rng, 0, lambda d, s: 0.0, lambda: (0, 0.0), lambda: 0.5, force_root=False))  # single leaf
    trees.append(synth._grow_tree(rng, 10, lambda d, s: 1.0 if s <= 0 else 0.0, lambda: (1, rng.normal()), lambda: rng.normal()))
    trees.append(synth._grow_tree(rng, 10, lambda d, s: 1.0 if s != 0 else 0.0, lambda: (2, rng.normal()), lambda: rng.normal()))
    path = tmp_path / "m.json"
    synth.write_xgboost_json(path, trees, 6)
    forest = model_io.load_xgboost_json(path)
    x = np.round(rng.normal(size=(400, 6)), 1).astype(np.float32)     # many values equal to thresholds
    tiled = cpu_oracle.TiledForest(forest, tile_size)
    np.testing.assert_array_equal(tiled.leaf_ids(x), cpu_oracle.leaf_ids(forest, x))
    pred, _ = cpu_oracle.predict(forest, x)
    np.testing.assert_allclose(tiled.predict_tree_outer(x, threads=3), pred, rtol=1e-5, atol=1e-5)


def test_tile_shapes_and_lut_known_answers():
    import math
    # left chain of three nodes (docs/TileShapesAndLUT/TileShapesAndLUT.md:36-46): node 0 -> left node 1 -> left node 2;
    # outcome strings there are written with node 0 first, the kernel word has node 0 in bit 0
    row = cpu_oracle.lut_for_shape([1, 2, -1], [-1, -1, -1], 3)
    word = lambda s: sum(int(c) << i for i, c in enumerate(s))
    assert row[word("110")] == 1 and row[word("111")] == 0
    assert all(row[word("0" + a + b)] == 3 for a in "01" for b in "01")        # root false: 4th child whatever the rest
    assert row[word("100")] == 2 and row[word("101")] == 2
    # complete tile of three nodes reduces to a textbook two-level descent
    row = cpu_oracle.lut_for_shape([1, -1, -1], [2, -1, -1], 3)
    for b0 in (0, 1):
        for b1 in (0, 1):
            for b2 in (0, 1):
                expected = (0 if b1 else 1) if b0 else (2 if b2 else 3)
                assert row[b0 | b1 << 1 | b2 << 2] == expected
    # number of tile shapes with exactly T nodes that random forests produce never exceeds Catalan(T), and for
    # small T a large sample hits every one of them (TileShapesAndLUT.md:15-19: 1, 2, 5, 14, ...)
    from treebeard_amd import synth
    rng = np.random.Generator(np.random.PCG64(99))
    trees = [synth._grow_tree(rng, 8, lambda d, s: 0.7, lambda: (rng.integers(0, 4), rng.normal()), lambda: rng.normal())
             for _ in range(400)]
    forest = model_io._assemble([(t.value, t.feature, t.left, t.right) for t in trees], num_features=4, initial_value=0.0,
                                transform=model_io.IDENTITY, num_classes=0, predicate=model_io.PRED_LT,
                                class_id=np.zeros(400, np.int32))
    for tile_size in (1, 2, 3, 4, 8):
        catalan = math.comb(2 * tile_size, tile_size) // (tile_size + 1)
        found = cpu_oracle.TiledForest(forest, tile_size).shapes_with_nodes(tile_size)
        assert found <= catalan
        if tile_size <= 4:
            assert found == catalan


def test_tiled_multithreaded_schedule_on_a_multiclass_forest(tmp_path, synth_model):
    """Class sums = the scalar walker's per-class sums (f32 order tolerance), class ids = the generated code's arg-max of
    them, exact ties included (two identical trees voting for classes 1 and 3: the larger id wins)."""
    forest = model_io.load_xgboost_json(synth_model(3))
    x = synth.CONFIGS[3].batch_rows(700, seed_offset=4)
    order = np.argsort([forest.depth(t) for t in range(forest.num_trees)], kind="stable").astype(np.int32)
    ids, sums = cpu_oracle.TiledForest(forest, 8).predict_tree_outer_multiclass(x, tree_order=order, threads=3)
    pred, margins = cpu_oracle.predict(forest, x)
    np.testing.assert_allclose(sums, margins, rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(ids, cpu_oracle.argmax_generated(sums))
    assert (ids == pred.astype(np.int8)).mean() > 0.999           # (f32 against f64 sums: only near-ties may differ)
    rng = np.random.Generator(np.random.PCG64(3))
    tree = synth._grow_tree(rng, 3, lambda d, s: 1.0, lambda: (int(rng.integers(0, 4)), float(np.round(rng.normal(), 1))),
                            lambda: float(rng.normal()))
    path = tmp_path / "ties.json"
    synth.write_xgboost_json(path, [tree, tree], 4, objective="multi:softmax", num_class=4, tree_info=[1, 3])
    tied = model_io.load_xgboost_json(path)
    rows = rng.normal(size=(64, 4)).astype(np.float32)
    ids, sums = cpu_oracle.TiledForest(tied, 8).predict_tree_outer_multiclass(rows, threads=2)
    np.testing.assert_array_equal(sums[:, 1], sums[:, 3])
    positive = sums[:, 1] > tied.initial_value
    np.testing.assert_array_equal(ids[positive], 3)                # classes 1 and 3 tie above the others: 3
    np.testing.assert_array_equal(ids[~positive & (sums[:, 1] < tied.initial_value)], 2)   # classes 0 and 2 tie at the initial value: 2


def test_tiled_multithreaded_schedule_matches_scalar_schedule():
    forest = model_io.load_xgboost_json(benchmark_model("airline"))
    x, _ = model_io.read_csv(benchmark_csv("airline"))
    x = x.astype(np.float32)
    order = np.argsort([forest.depth(t) for t in range(forest.num_trees)], kind="stable").astype(np.int32)
    scalar = cpu_oracle.predict_tree_outer(forest, x, tree_order=order, threads=2)
    tiled = cpu_oracle.TiledForest(forest, 8).predict_tree_outer(x, tree_order=order, threads=5)
    np.testing.assert_array_equal(tiled, scalar)     # same leaves, same f32 summation order

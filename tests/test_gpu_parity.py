"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real GPU.

Bars: per-tree leaf selection bit-exact; predictions within 1e-5 relative of the
oracle (sums) and 1e-6 absolute (sigmoid / softmax); class ids equal.  At the
full benchmark sizes the whole batch is compared with the oracle when the host
has at least 8 threads to split the rows over (a random sample of rows
otherwise), next to size-independent properties (sub-batch consistency,
permutation equivariance).
"""
import ctypes
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle, model_io  # noqa: E402
from treebeard_amd import synth, treebeard  # noqa: E402
from treebeard_amd.runtime_api import api  # noqa: E402

from conftest import BENCHMARK_XGB, GOLDEN, benchmark_csv, benchmark_model, random_models  # noqa: E402
from onnx_writer import write_onnx  # noqa: E402

RTOL_SUM = 1e-5
ATOL_PROB = 1e-6


@pytest.fixture(scope="module", autouse=True)
def require_gpu():
    assert api().runtime_lib.tbmi_device_count() >= 1, "the GPU tests need a HIP device"
    assert torch.cuda.is_available()


def make_runner(path, batch, kind="xgboost_json", num_features=0, gpu_options=None, float_class_ids=False):
    options = treebeard.CompilerOptions(batch, 1)
    if num_features:
        options.SetNumberOfFeatures(num_features)
    if not float_class_ids and is_multiclass(path, kind, num_features):
        options.SetReturnTypeWidth(8)                  # what the reference's multiclass tests set
        options.SetReturnTypeIsFloatType(False)        # (test/python/cpu_tests.py:20-22)
    ctx = treebeard.TreebeardContext(str(path), "", options, gpu_options)
    ctx.SetInputFiletype(kind)
    ctx.SetRepresentationType("gpu_sparse")
    return treebeard.TreebeardInferenceRunner.GPUInferenceRunnerFromTBContext(ctx)


def is_multiclass(path, kind, num_features):
    lib = api().runtime_lib
    h = lib.tbmi_load_forest(str(path).encode(), kind.encode(), num_features)
    assert h, api().last_error()
    info = (ctypes.c_int64 * 6)()
    initial = ctypes.c_double()
    assert lib.tbmi_forest_info(h, info, ctypes.byref(initial)) == 0
    lib.tbmi_delete_forest(h)
    return info[2] > 0


def gpu_predict(runner, x):
    dx = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).cuda()
    rows = x.shape[0]
    if runner.result_dtype() == np.int8:
        out = torch.full((rows,), -1, dtype=torch.int8, device="cuda")
    else:
        out = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
    runner.run_device(dx.data_ptr(), out.data_ptr(), rows)
    return out.cpu().numpy()


def gpu_leaf_ids(runner, x):
    dx = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).cuda()
    ids = torch.full((x.shape[0], runner.num_trees()), -7, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
    runner.dump_leaf_ids(dx.data_ptr(), ids.data_ptr(), x.shape[0])
    return ids.cpu().numpy()


def check_against_oracle(runner, forest, x):
    np.testing.assert_array_equal(gpu_leaf_ids(runner, x), cpu_oracle.leaf_ids(forest, x))
    pred, sums = cpu_oracle.predict(forest, x)
    got = gpu_predict(runner, x)
    if forest.num_classes > 0:
        voted = np.isin(np.arange(forest.num_classes), forest.class_id)
        if not voted.all():
            # a class without trees scores the initial value, as in the reference's generated code
            # (test_classes_without_trees_score_the_initial_value states the two reference behaviours)
            margins = np.where(voted[None, :], sums, forest.initial_value).astype(np.float32)
            pred = cpu_oracle.argmax_generated(margins).astype(np.float32)
        np.testing.assert_array_equal(got.astype(np.float32), pred)
    elif forest.transform == model_io.SIGMOID:
        np.testing.assert_allclose(got, pred, rtol=0, atol=ATOL_PROB)
    else:
        np.testing.assert_allclose(got, pred, rtol=RTOL_SUM, atol=0)
    return got


# --------------------------------------------------------------------------
# the reference's own fixtures
# --------------------------------------------------------------------------
@pytest.mark.parametrize("path", random_models(), ids=os.path.basename)
def test_random_models(path):
    forest = model_io.load_xgboost_json(path)
    x, expected = model_io.read_csv(path + ".csv")
    x = x.astype(np.float32)
    runner = make_runner(path, x.shape[0])
    got = check_against_oracle(runner, forest, x)
    np.testing.assert_allclose(got, expected, rtol=2e-5, atol=2e-5)   # XGBoost's own f32-accumulated output
    # host-buffer entry point, as the reference's tests drive it (batch = whole CSV)
    np.testing.assert_array_equal(runner.RunInference(x), got)


@pytest.mark.parametrize("name", BENCHMARK_XGB)
def test_benchmark_models(name, plain_file):
    forest = model_io.load_xgboost_json(benchmark_model(name))
    x, expected = model_io.read_csv(benchmark_csv(name))
    x = x.astype(np.float32)
    runner = make_runner(plain_file(benchmark_model(name)), 100)
    got = check_against_oracle(runner, forest, x)
    if forest.transform == model_io.SIGMOID:
        np.testing.assert_allclose(got, expected, rtol=0, atol=ATOL_PROB)
    else:
        np.testing.assert_allclose(got, expected, rtol=RTOL_SUM, atol=0)
    # 200 rows = 2 batches of 100 (the reference's python tests feed fixed batches)
    np.testing.assert_array_equal(runner.RunInferenceOnMultipleBatches(x), got)


def test_onnx_abalone(plain_file):
    path = os.path.join(GOLDEN, "benchmark", "abalone_onnx_model_save.onnx.gz")
    forest = model_io.load_onnx(path, 8)
    x, expected = model_io.read_csv(os.path.join(GOLDEN, "benchmark", "abalone_onnx_model_save.onnx.csv"))
    x = x.astype(np.float32)
    options = treebeard.CompilerOptions(x.shape[0], 1)
    options.SetNumberOfFeatures(8)
    runner = treebeard.TreebeardInferenceRunner.FromONNXModelFile(plain_file(path), options)
    got = check_against_oracle(runner, forest, x)
    np.testing.assert_allclose(got, expected, rtol=RTOL_SUM, atol=0)


@pytest.mark.parametrize("mode", ["BRANCH_LT", "BRANCH_GEQ", "BRANCH_GT", "BRANCH_LEQ"])
def test_onnx_comparison_modes(tmp_path, mode):
    rng = np.random.default_rng(11)
    trees = []
    for _ in range(9):
        thr = rng.integers(-3, 4, size=7).astype(np.float32) / 2      # coarse grid: x == threshold happens
        trees.append((thr, rng.integers(0, 4, 7), [1, 3, 5, -1, -1, -1, -1], [2, 4, 6, -1, -1, -1, -1]))
    path = tmp_path / "m.onnx"
    write_onnx(path, trees, mode=mode, base_value=0.5)
    forest = model_io.load_onnx(path, 4)
    x = (rng.integers(-4, 5, size=(777, 4)) / 2).astype(np.float32)
    runner = make_runner(path, 777, "onnx_file", 4)
    check_against_oracle(runner, forest, x)


@pytest.mark.parametrize("slices", [1, 2])
@pytest.mark.parametrize("post_transform", ["NONE", "LOGISTIC", "SOFTMAX"])
def test_onnx_classifier(tmp_path, post_transform, slices):
    """TreeEnsembleClassifier through the ONNX loader (src/json/onnxmodelparser.h:102-113, :162-172, :355-374):
    one class id per tree, any post_transform; leaf ids and class ids against the oracle on the forest its own
    loader reads, with leaf weights on a coarse grid so that class sums tie exactly on many rows (the larger
    class id wins, src/reduction/LowerReduceOps.cpp:148-187), on the walk kernel's own arg-max (one tree slice)
    and through the finalize kernel (two)."""
    rng = np.random.Generator(np.random.PCG64(77))
    classes, features = 6, 5
    split = lambda: (rng.integers(0, features), rng.normal())
    grown = [synth._grow_tree(rng, 4, lambda d, s: 0.8, split, lambda: float(rng.integers(-2, 3)) * 0.25) for _ in range(40)]
    trees = [(np.asarray(t.value, np.float32), t.feature, t.left, t.right) for t in grown]
    class_ids = [int(c) for c in rng.integers(0, classes - 1, len(trees))]           # the last class gets no tree
    path = tmp_path / "classifier.onnx"
    write_onnx(path, trees, base_value=0.25, post_transform=post_transform, classifier=True, n_classes=classes, class_ids=class_ids)
    forest = model_io.load_onnx(path, features)
    assert forest.num_classes == classes and list(forest.class_id) == class_ids
    rows = 1500
    x = rng.normal(size=(rows, features)).astype(np.float32)
    runner = make_runner(path, rows, "onnx_file", features)
    assert runner.result_dtype() == np.int8
    runner.set_plan(64, 2, 2, 4096, slices)
    got = check_against_oracle(runner, forest, x)
    _, sums = cpu_oracle.predict(forest, x)
    best = sums.max(axis=1, keepdims=True)
    assert ((sums == best).sum(axis=1) > 1).sum() > 20          # exact ties for the maximum do occur
    ties = (sums[:, :classes - 1] == best).sum(axis=1) > 1
    voted = np.where(sums[:, :classes - 1] == best, np.arange(classes - 1)[None, :], -1).max(axis=1)
    unvoted_wins = 0.25 >= best[:, 0]                           # the class without trees scores the base value
    np.testing.assert_array_equal(got[ties & ~unvoted_wins], voted[ties & ~unvoted_wins])


def test_onnx_classifier_with_several_class_ids_in_one_tree_is_refused(tmp_path):
    rng = np.random.Generator(np.random.PCG64(78))
    grown = [synth._grow_tree(rng, 3, lambda d, s: 0.9, lambda: (rng.integers(0, 3), rng.normal()), lambda: rng.normal()) for _ in range(3)]
    trees = [(np.asarray(t.value, np.float32), t.feature, t.left, t.right) for t in grown]
    path = tmp_path / "mixed.onnx"
    write_onnx(path, trees, classifier=True, n_classes=3, class_ids=[0, [1, 2], 2])
    options = treebeard.CompilerOptions(64, 1)
    options.SetNumberOfFeatures(3)
    with pytest.raises(RuntimeError, match="multiple class IDs per tree"):
        treebeard.TreebeardInferenceRunner.FromONNXModelFile(str(path), options)


# --------------------------------------------------------------------------
# the benchmark configurations at oracle-sized batches
# --------------------------------------------------------------------------
@pytest.mark.parametrize("k,rows", [(1, 1024), (2, 4096), (3, 4096), (4, 512), (5, 4096)])
def test_synthetic_configurations(synth_model, k, rows):
    forest = model_io.load_xgboost_json(synth_model(k))
    x = synth.CONFIGS[k].batch_rows(rows)
    runner = make_runner(synth_model(k), rows)
    check_against_oracle(runner, forest, x)
    if k == 3:
        dx = torch.from_numpy(x).cuda()
        cls = torch.zeros(rows, dtype=torch.int8, device="cuda")
        margins = torch.zeros((rows, 8), dtype=torch.float32, device="cuda")
        probs = torch.zeros((rows, 8), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
        runner.run_device_multiclass(dx.data_ptr(), rows, cls.data_ptr(), margins.data_ptr(), probs.data_ptr())
        pred, sums = cpu_oracle.predict(forest, x)
        np.testing.assert_allclose(margins.cpu().numpy(), sums, rtol=RTOL_SUM, atol=1e-7)
        # softmax probabilities: closed form only (the reference never computes them)
        np.testing.assert_allclose(probs.cpu().numpy(), cpu_oracle.softmax(sums), rtol=0, atol=ATOL_PROB)
        np.testing.assert_array_equal(cls.cpu().numpy(), cpu_oracle.argmax_generated(sums.astype(np.float32)))


@pytest.mark.parametrize("rows", [1, 64, 4096, 1 << 16])
def test_config2_batch_sweep(synth_model, rows):
    forest = model_io.load_xgboost_json(synth_model(2))
    x = synth.CONFIGS[2].batch_rows(rows, seed_offset=rows)
    runner = make_runner(synth_model(2), rows)
    if rows <= 4096:
        check_against_oracle(runner, forest, x)
    else:
        pred, _ = cpu_oracle.predict(forest, x)
        np.testing.assert_allclose(gpu_predict(runner, x), pred, rtol=0, atol=ATOL_PROB)


@pytest.mark.parametrize("k", [2, 3, 5, 4])
def test_full_size_properties(synth_model, k):
    cfg = synth.CONFIGS[k]
    rows = cfg.batch
    forest = model_io.load_xgboost_json(synth_model(k))
    x = cfg.batch_rows(rows)
    runner = make_runner(synth_model(k), rows)
    full = gpu_predict(runner, x)
    assert not np.isnan(full.astype(np.float32)).any()
    rng = np.random.default_rng(k)
    # (1) every row against the oracle when the host has the cores to walk the whole batch in seconds
    # (rows split over the threads), else a random sample of rows
    threads = cpu_oracle.max_threads()
    pick = slice(None) if threads >= 8 else rng.choice(rows, size=4096, replace=False)
    pred, _ = cpu_oracle.predict(forest, x if threads >= 8 else x[pick], threads=threads)
    if forest.num_classes > 0:
        np.testing.assert_array_equal(full[pick].astype(np.float32), pred)
    elif forest.transform == model_io.SIGMOID:
        np.testing.assert_allclose(full[pick], pred, rtol=0, atol=ATOL_PROB)
    else:
        np.testing.assert_allclose(full[pick], pred, rtol=RTOL_SUM, atol=0)
    # (2) rows are independent: a ragged slice alone gives the same bits as inside the batch
    lo, hi = 12345, 12345 + 70001
    np.testing.assert_array_equal(gpu_predict(runner, x[lo:hi]), full[lo:hi])
    # (3) permutation equivariance
    perm = rng.permutation(rows)
    np.testing.assert_array_equal(gpu_predict(runner, x[perm]), full[perm])


# --------------------------------------------------------------------------
# launch plans, edge cases, API behaviour
# --------------------------------------------------------------------------
@pytest.mark.parametrize("plan", [(64, 1, 1, 16384, 1), (128, 1, 2, 32768, 3), (256, 1, 8, 65536, 1), (512, 1, 4, 49152, 5),
                                  (256, 1, 4, 8192, 40), (256, 4, 4, 65536, 1), (128, 8, 2, 40960, 2), (64, 3, 1, 16384, 1),
                                  (512, 2, 8, 32768, 1)])
@pytest.mark.parametrize("k", [2, 3])
def test_launch_plans_agree(synth_model, k, plan):
    if k == 3 and plan[0] == 512:
        pytest.skip("54 features x 512 rows exceed the LDS row tile")
    forest = model_io.load_xgboost_json(synth_model(k))
    x = synth.CONFIGS[k].batch_rows(3001, seed_offset=9)
    runner = make_runner(synth_model(k), 3001)
    runner.set_plan(*plan)
    assert "kernel=rows_lds rowsPerBlock=%d treeThreads=%d treeLanes=1 interleave=%d" % plan[:3] in runner.describe_plan()
    # both ways of bringing tree groups into LDS: through prefetch registers, and by direct global-to-LDS copies
    results = []
    for mode, name in ((1, "registers"), (2, "direct")):
        runner.set_group_staging(mode)
        assert "staging=" + name in runner.describe_plan()
        results.append(check_against_oracle(runner, forest, x))
    np.testing.assert_array_equal(results[0], results[1])


@pytest.mark.parametrize("k", [1, 2, 3, 4, 5])
def test_group_staging_follows_the_blocks_per_compute_unit(synth_model, k):
    """By rule tree groups are copied straight into LDS when two blocks fit a compute unit (one walks while the
    other waits for its copy) and go through prefetch registers otherwise; either way the results are the same."""
    cfg = synth.CONFIGS[k]
    rows = 1 << 16 if k != 4 else 1 << 12       # (enough row blocks for one tree slice)
    forest = model_io.load_xgboost_json(synth_model(k))
    x = cfg.batch_rows(rows, seed_offset=21)
    runner = make_runner(synth_model(k), rows)
    plan = runner.describe_plan()
    if "kernel=rows_lds" not in plan:
        pytest.skip("the automatic plan for this batch is not the row-parallel kernel: " + plan)
    lds = int(plan.split("ldsBytes=")[1].split()[0])
    assert ("staging=direct" in plan) == (2 * (lds + 512) <= 160 * 1024), plan
    by_rule = gpu_predict(runner, x)
    for mode in (1, 2):
        runner.set_group_staging(mode)
        np.testing.assert_array_equal(gpu_predict(runner, x), by_rule)
    runner.set_group_staging(0)
    sample = slice(0, 2048)
    np.testing.assert_array_equal(gpu_leaf_ids(runner, x[sample]), cpu_oracle.leaf_ids(forest, x[sample]))
    with pytest.raises(RuntimeError):
        runner.set_group_staging(3)


@pytest.mark.parametrize("plan", [(1, 256, 1, 0, 0), (4, 64, 1, 32768, 7), (16, 16, 2, 0, 1), (2, 128, 1, 16384, 0),
                                  (8, 8, 4, 0, 3), (64, 1, 1, 0, 2), (1, 1024, 1, 65536, 1)])
@pytest.mark.parametrize("k", [2, 3])
def test_tree_parallel_plans_agree(synth_model, k, plan):
    forest = model_io.load_xgboost_json(synth_model(k))
    x = synth.CONFIGS[k].batch_rows(203, seed_offset=3)
    runner = make_runner(synth_model(k), 203)
    runner.set_tree_parallel_plan(*plan)
    assert "kernel=tree_parallel rowsPerBlock=%d treeThreads=1 treeLanes=%d" % plan[:2] in runner.describe_plan()
    check_against_oracle(runner, forest, x)


@pytest.mark.parametrize("k,rows", [(3, 100), (5, 7), (1, 1)])
def test_small_batches_pick_the_tree_parallel_kernel(synth_model, k, rows):
    forest = model_io.load_xgboost_json(synth_model(k))
    x = synth.CONFIGS[k].batch_rows(rows, seed_offset=1)
    runner = make_runner(synth_model(k), rows)
    assert "kernel=tree_parallel" in runner.describe_plan()
    check_against_oracle(runner, forest, x)


def coarse_model(path, num_features, num_trees, num_class, seed):
    """Trees whose thresholds come from a grid of 40 values per feature (so ranks fit one byte)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    grid = np.round(rng.normal(size=(40, num_features)), 2).astype(np.float32)
    trees = [synth._grow_tree(rng, 7, lambda d, s: 0.85, lambda: (lambda f: (f, grid[rng.integers(0, 40), f]))(rng.integers(0, num_features)),
                              lambda: rng.normal(0, 0.1)) for _ in range(num_trees)]
    synth.write_xgboost_json(path, trees, num_features, objective="multi:softmax" if num_class else "reg:squarederror",
                             num_class=num_class, tree_info=[t % num_class for t in range(num_trees)] if num_class else None)
    return grid


@pytest.mark.parametrize("plan", [(8, 4, 0, 1), (16, 1, 16384, 1), (4, 2, 32768, 3), (1, 8, 16384, 1)])
@pytest.mark.parametrize("model", ["config4", "coarse_regression", "coarse_multiclass"])
def test_rank_quantised_plans_agree(synth_model, tmp_path, model, plan):
    """Rows replaced by one-byte ranks among each feature's thresholds: leaf selection must not change."""
    if model == "config4":
        path, rows = synth_model(4), 333
        x = synth.CONFIGS[4].batch_rows(rows, seed_offset=5)
    else:
        path, rows = str(tmp_path / "coarse.json"), 1500
        grid = coarse_model(path, 37, 120, 5 if model == "coarse_multiclass" else 0, seed=17)
        rng = np.random.default_rng(3)
        x = np.round(rng.normal(size=(rows, 37)), 2).astype(np.float32)     # many values equal to thresholds
    forest = model_io.load_xgboost_json(path)
    thr, feat, left, _ = forest.tree(0)
    for i in np.nonzero(left != -1)[0][:20]:
        x[int(i) % rows, feat[i]] = np.float32(thr[i])
    x[3, :] = np.inf
    x[4, :] = -np.inf
    runner = make_runner(path, rows)
    runner.set_quantized_plan(*plan)
    assert "quantizedRows=1" in runner.describe_plan()
    check_against_oracle(runner, forest, x)


@pytest.mark.parametrize("plan", [(256, 4, 4, 0, 1), (512, 2, 4, 32768, 1), (128, 8, 2, 16384, 3), (64, 1, 1, 16384, 2), (1024, 1, 8, 16384, 1)])
@pytest.mark.parametrize("model", ["config2", "config3", "config5", "coarse_regression", "coarse_multiclass"])
def test_two_byte_rank_plans_agree(synth_model, tmp_path, model, plan):
    """Rows replaced by two-byte ranks among each feature's thresholds (a ranking kernel in front of the walk, tile
    [feature pair][row][2]): leaf selection must not change - even and odd feature counts, values that sit on
    thresholds, +-inf and NaN, regressors and classifiers, several block shapes and tree slices."""
    if model.startswith("config"):
        k = int(model[-1])
        path, rows = synth_model(k), 2500
        x = synth.CONFIGS[k].batch_rows(rows, seed_offset=5)
    else:
        path, rows = str(tmp_path / "coarse.json"), 1500
        coarse_model(path, 37, 120, 5 if model == "coarse_multiclass" else 0, seed=17)       # 37 features: the pad slot shares the last pair
        rng = np.random.default_rng(3)
        x = np.round(rng.normal(size=(rows, 37)), 2).astype(np.float32)     # many values equal to thresholds
    forest = model_io.load_xgboost_json(path)
    thr, feat, left, _ = forest.tree(0)
    for i in np.nonzero(left != -1)[0][:20]:
        x[int(i) % rows, feat[i]] = np.float32(thr[i])
        x[(int(i) + 50) % rows, feat[i]] = np.nextafter(np.float32(thr[i]), np.float32(-np.inf))
    x[3, :] = np.inf
    x[4, :] = -np.inf
    x[5, ::2] = np.nan
    runner = make_runner(path, rows)
    if plan[0] * ((forest.num_features + 2) // 2) * 4 > 65536:
        with pytest.raises(RuntimeError, match="below 64 KB|do not fit 16 bits"):
            runner.set_rank16_plan(*plan)
        return
    runner.set_rank16_plan(*plan)
    assert "rankRows16=1" in runner.describe_plan() and "staging=direct" in runner.describe_plan()
    check_against_oracle(runner, forest, x)
    # the other entry points on the same plan: host buffers, the caller's stream, no allocation
    expected = gpu_predict(runner, x)
    np.testing.assert_array_equal(runner.RunInference(x, runner.result_dtype()), expected)
    dx = torch.from_numpy(x).cuda()
    got = torch.zeros(rows, dtype=torch.int8 if runner.result_dtype() == np.int8 else torch.float32, device="cuda")
    stream = torch.cuda.current_stream()
    runner.run_device_noalloc(dx.data_ptr(), got.data_ptr(), rows, stream.cuda_stream)
    stream.synchronize()
    np.testing.assert_array_equal(got.cpu().numpy(), expected)


def test_two_byte_rank_plan_survives_the_compiled_model_file(synth_model, tmp_path):
    forest = model_io.load_xgboost_json(synth_model(5))
    x = synth.CONFIGS[5].batch_rows(3000, seed_offset=2)
    runner = make_runner(synth_model(5), 3000)
    runner.set_rank16_plan(256, 4, 8, 32768, 1)
    path = str(tmp_path / "rank16.tbamd")
    runner.save_compiled_model(path)
    again = treebeard.TreebeardInferenceRunner.FromSOFile(path, "")
    assert again.describe_plan() == runner.describe_plan() and "rankRows16=1" in again.describe_plan()
    check_against_oracle(again, forest, x)


def test_rank_quantisation_is_refused_when_a_feature_has_too_many_thresholds(synth_model):
    runner = make_runner(synth_model(2), 512)
    with pytest.raises(RuntimeError, match="254 distinct thresholds"):
        runner.set_quantized_plan(8, 4, 0, 1)


def test_gpu_auto_schedule_options_are_honoured(synth_model):
    gpu = treebeard.GPUAutoScheduleOptions.Construct(num_rows_per_TB=64, num_tree_threads=10,
                                                     tree_walk_interleave_factor=2, cache_rows=True)
    runner = make_runner(synth_model(1), 1024, gpu_options=gpu)
    plan = runner.describe_plan()
    assert "kernel=rows_lds rowsPerBlock=64 " in plan and "interleave=2" in plan
    forest = model_io.load_xgboost_json(synth_model(1))
    check_against_oracle(runner, forest, synth.CONFIGS[1].batch_rows(1024))


def test_autotuned_runner_matches(synth_model):
    options = treebeard.CompilerOptions(8192, 1)
    ctx = treebeard.TreebeardContext(synth_model(1), "", options)
    runner = treebeard.TreebeardInferenceRunner.AutoScheduleGPUInferenceRunnerFromTBContext(ctx)
    forest = model_io.load_xgboost_json(synth_model(1))
    check_against_oracle(runner, forest, synth.CONFIGS[1].batch_rows(8192))


def test_degenerate_models(tmp_path):
    rng = np.random.Generator(np.random.PCG64(4))
    stump = synth._grow_tree(rng, 0, lambda d, s: 0.0, lambda: (0, 0.0), lambda: 0.75, force_root=False)   # single leaf
    deep = synth._grow_tree(rng, 9, lambda d, s: 1.0 if s <= 0 else 0.0, lambda: (rng.integers(0, 3), rng.normal()),
                            lambda: rng.normal())                                                         # left spine
    one = synth._grow_tree(rng, 1, lambda d, s: 1.0, lambda: (1, 0.0), lambda: rng.normal())
    for name, trees in (("stump", [stump]), ("mixed", [stump, deep, one, stump]), ("one", [one])):
        path = tmp_path / (name + ".json")
        synth.write_xgboost_json(path, trees, 3)
        forest = model_io.load_xgboost_json(path)
        x = rng.normal(size=(130, 3)).astype(np.float32)
        x[5, 1] = 0.0          # equal to a threshold
        x[7, :] = np.inf
        x[8, :] = -np.inf
        check_against_oracle(make_runner(path, 130), forest, x)


def test_zero_rows_and_errors(synth_model):
    runner = make_runner(synth_model(1), 16)
    torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
    runner.run_device(None, None, 0)
    lib = api().runtime_lib
    assert lib.tbmi_run_device(0, None, None, 4) == -1 and "null" in api().last_error()
    options = treebeard.CompilerOptions(16, 1)
    options.SetInputElementTypeWidth(64)
    with pytest.raises(RuntimeError, match="32-bit float inputs"):
        treebeard.TreebeardInferenceRunner.FromModelFile(synth_model(1), "", options)
    with pytest.raises(RuntimeError, match="cannot open"):
        treebeard.TreebeardInferenceRunner.FromModelFile("/nonexistent.json", "", treebeard.CompilerOptions(16, 1))


def test_kernel_time_shim(synth_model):
    runner = make_runner(synth_model(1), 1024)
    x = synth.CONFIGS[1].batch_rows(1024)
    treebeard.SetEnableMeasureGpuKernelTime(True)
    treebeard.SetNumberOfKernelRuns(10)
    try:
        runner.RunInference(x)
        ten = treebeard.GetGPUKernelExecutionTime(runner)
        treebeard.SetNumberOfKernelRuns(1)
        runner.RunInference(x)
        one = treebeard.GetGPUKernelExecutionTime(runner)
    finally:
        treebeard.SetEnableMeasureGpuKernelTime(False)
        treebeard.SetNumberOfKernelRuns(1)
    assert ten > one > 0
    dx = torch.from_numpy(x).cuda()
    out = torch.zeros(1024, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
    walk_ms, fin_ms = runner.time_kernels(dx.data_ptr(), out.data_ptr(), 1024, 5)
    assert 0 < walk_ms < 50 and fin_ms >= 0


@pytest.mark.parametrize("rows", [1, 3, 63, 64, 65, 255, 257, 1000])
@pytest.mark.parametrize("features,offset", [(3, 0), (5, 1), (28, 0), (28, 3), (33, 2)])
def test_row_staging_alignment_and_ragged_tails(tmp_path, rows, features, offset):
    """Inputs that start off a 16-byte boundary, odd feature counts and batches that end inside a block."""
    rng = np.random.Generator(np.random.PCG64(features * 1000 + rows))
    trees = [synth._grow_tree(rng, 5, lambda d, s: 0.9, lambda: (rng.integers(0, features), rng.normal()),
                              lambda: rng.normal()) for _ in range(20)]
    path = tmp_path / "m.json"
    synth.write_xgboost_json(path, trees, features)
    forest = model_io.load_xgboost_json(path)
    x = rng.normal(size=(rows, features)).astype(np.float32)
    expected, _ = cpu_oracle.predict(forest, x)
    flat = torch.zeros(rows * features + 8, dtype=torch.float32, device="cuda")
    flat[offset:offset + rows * features] = torch.from_numpy(x.reshape(-1)).cuda()
    out = torch.zeros(rows, dtype=torch.float32, device="cuda")
    for setup in (lambda r: None, lambda r: r.set_plan(64, 2, 2, 16384, 1), lambda r: r.set_tree_parallel_plan(4, 16, 1, 16384, 1)):
        runner = make_runner(path, rows)
        setup(runner)
        out.fill_(float("nan"))
        torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
        runner.run_device(flat.data_ptr() + 4 * offset, out.data_ptr(), rows)
        np.testing.assert_allclose(out.cpu().numpy(), expected, rtol=RTOL_SUM, atol=0)


@pytest.mark.parametrize("k,rows", [(2, (1 << 18) + 777), (3, 1 << 17), (4, 5000)])
def test_host_buffer_entry_point_pipelines_large_batches(synth_model, k, rows):
    """RunInference on host memory copies and computes a large batch in overlapping pieces: same bits as one launch."""
    x = synth.CONFIGS[k].batch_rows(rows, seed_offset=2)
    runner = make_runner(synth_model(k), rows)
    device = gpu_predict(runner, x)
    host = runner.RunInference(x, resultType=runner.result_dtype())              # pageable: staged through pinned buffers
    np.testing.assert_array_equal(host, device)
    np.testing.assert_array_equal(runner.RunInference(x, resultType=runner.result_dtype()), device)   # buffers reused
    pinned = torch.from_numpy(x).pin_memory()                                        # pinned: read by DMA where it lies
    np.testing.assert_array_equal(runner.RunInference(pinned.numpy(), resultType=runner.result_dtype()), device)
    forest = model_io.load_xgboost_json(synth_model(k))
    pick = np.random.default_rng(k).choice(rows, size=2048, replace=False)
    pred, _ = cpu_oracle.predict(forest, x[pick])
    if forest.num_classes > 0:
        np.testing.assert_array_equal(host[pick].astype(np.float32), pred)
    elif forest.transform == model_io.SIGMOID:
        np.testing.assert_allclose(host[pick], pred, rtol=0, atol=ATOL_PROB)
    else:
        np.testing.assert_allclose(host[pick], pred, rtol=RTOL_SUM, atol=0)


@pytest.mark.parametrize("k", [2, 3, 4])
def test_compiled_model_file_round_trip(synth_model, tmp_path, k):
    """Compile once, reload: the saved file reopens without the source model and predicts the same bits."""
    rows = 2000
    x = synth.CONFIGS[k].batch_rows(rows, seed_offset=4)
    runner = make_runner(synth_model(k), rows)
    if k == 2:
        runner.set_plan(128, 8, 2, 32768, 3)
    expected = gpu_predict(runner, x)
    path = str(tmp_path / "model.tbamd")
    runner.save_compiled_model(path)
    plan = runner.describe_plan()
    del runner
    reopened = treebeard.TreebeardInferenceRunner.FromCompiledModelFile(path)
    assert reopened.batchSize == rows and reopened.describe_plan() == plan
    np.testing.assert_array_equal(gpu_predict(reopened, x), expected)
    forest = model_io.load_xgboost_json(synth_model(k))
    np.testing.assert_array_equal(gpu_leaf_ids(reopened, x[:256]), cpu_oracle.leaf_ids(forest, x[:256]))
    # the reference's own entry point for reopening a compiled model (src/runtime/runtime.cpp:35-54, FromSOFile)
    again = treebeard.TreebeardInferenceRunner.FromSOFile(path, str(tmp_path / "globals.json"))
    assert again.batchSize == rows and again.rowSize == forest.num_features and again.describe_plan() == plan
    check_against_oracle(again, forest, x)
    np.testing.assert_array_equal(again.RunInference(x, again.result_dtype()), expected)
    with pytest.raises(RuntimeError, match="InitializeInferenceRunner"):
        treebeard.TreebeardInferenceRunner.FromSOFile(str(tmp_path / "missing.tbamd"), "")
    with open(path, "r+b") as fh:
        fh.truncate(os.path.getsize(path) // 2)
    with pytest.raises(RuntimeError, match="truncated"):
        treebeard.TreebeardInferenceRunner.FromCompiledModelFile(path)


@pytest.mark.parametrize("paths", ["default", "rows_lds", "tree_parallel", "quantised"])
def test_nan_inputs_follow_the_scalar_walk(tmp_path, paths):
    """NaN compares false, so a NaN feature sends the row to the right child (src/include/DecisionForest.h:372-375)."""
    path = str(tmp_path / "coarse.json")
    coarse_model(path, 9, 40, 0, seed=23)
    forest = model_io.load_xgboost_json(path)
    rng = np.random.default_rng(8)
    x = np.round(rng.normal(size=(300, 9)), 2).astype(np.float32)
    x[rng.random(x.shape) < 0.2] = np.nan
    runner = make_runner(path, 300)
    if paths == "rows_lds":
        runner.set_plan(64, 2, 2, 16384, 2)
    elif paths == "tree_parallel":
        runner.set_tree_parallel_plan(4, 16, 1, 16384, 3)
    elif paths == "quantised":
        runner.set_quantized_plan(4, 2, 16384, 1)
    check_against_oracle(runner, forest, x)


@pytest.mark.parametrize("k,rows,slices", [(2, 3, 40), (3, 50, 24), (1, 700, 20)])
def test_many_tree_slices_on_small_batches(synth_model, k, rows, slices):
    """Few rows spread over many tree slices: the wave-per-row finalize adds the slices."""
    forest = model_io.load_xgboost_json(synth_model(k))
    x = synth.CONFIGS[k].batch_rows(rows, seed_offset=6)
    runner = make_runner(synth_model(k), rows)
    runner.set_plan(64, 2, 1, 4096 if k != 5 else 16384, slices)
    assert "treeSlices=%d" % slices in runner.describe_plan()
    check_against_oracle(runner, forest, x)
    if k == 3:
        dx = torch.from_numpy(x).cuda()
        margins = torch.zeros((rows, 8), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
        runner.run_device_multiclass(dx.data_ptr(), rows, None, margins.data_ptr(), None)
        np.testing.assert_allclose(margins.cpu().numpy(), cpu_oracle.predict(forest, x)[1], rtol=RTOL_SUM, atol=1e-7)


# --------------------------------------------------------------------------
# forests with a tree too big for an LDS tree group: the global-memory walk
# --------------------------------------------------------------------------
def big_tree_model(path, num_class, seed=21):
    rng = np.random.Generator(np.random.PCG64(seed))
    split = lambda: (rng.integers(0, 12), rng.normal())
    leaf = lambda: rng.normal(0.0, 0.1)
    trees = [synth._grow_tree(rng, 14, lambda d, s: 1.0 if d < 13 else 0.6, split, leaf)]        # > 8190 nodes
    trees += [synth._grow_tree(rng, int(rng.integers(0, 9)), lambda d, s: 0.8, split, leaf, force_root=False)
              for _ in range(37)]
    if num_class:
        info = [int(c) for c in rng.permutation(len(trees)) % num_class]                         # every class has trees
        synth.write_xgboost_json(path, trees, 12, objective="multi:softmax", num_class=num_class, tree_info=info)
    else:
        synth.write_xgboost_json(path, trees, 12, objective="binary:logistic")
    return path


@pytest.mark.parametrize("num_class", [0, 6])
@pytest.mark.parametrize("rows", [1, 77, 5000])
def test_trees_too_big_for_lds_walk_from_global_memory(tmp_path, num_class, rows):
    path = big_tree_model(tmp_path / "big.json", num_class)
    forest = model_io.load_xgboost_json(path)
    assert max(len(forest.tree(t)[0]) for t in range(forest.num_trees)) > 8190
    x = np.random.Generator(np.random.PCG64(rows)).normal(size=(rows, 12)).astype(np.float32)
    runner = make_runner(path, rows)
    assert "kernel=global_walk" in runner.describe_plan()
    check_against_oracle(runner, forest, x)
    with pytest.raises(RuntimeError, match="does not fit"):
        runner.set_plan(256, 1, 4, 65536, 1)


@pytest.mark.parametrize("plan", [(64, 1, 1), (256, 2, 7), (1024, 8, 3), (128, 4, 1000)])
@pytest.mark.parametrize("k", [1, 3])
def test_global_walk_plans_agree(synth_model, k, plan):
    forest = model_io.load_xgboost_json(synth_model(k))
    x = synth.CONFIGS[k].batch_rows(1500, seed_offset=6)
    runner = make_runner(synth_model(k), 1500)
    runner.set_global_walk_plan(*plan)
    assert "kernel=global_walk rowsPerBlock=%d" % plan[0] in runner.describe_plan()
    check_against_oracle(runner, forest, x)


@pytest.mark.parametrize("kernel", ["rows_lds", "rows_lds_one_slice", "tree_parallel", "global_walk"])
def test_classes_without_trees_score_the_initial_value(tmp_path, kernel):
    """The reference's two sides disagree on a class no tree votes for: its generated code fills every class
    sum with the initial value before reducing (src/reduction/LowerReduceOps.cpp:1459-1470,
    src/mlir/LowerToMidLevelIR.cpp:405-428), its scalar check leaves such a class at 0
    (src/include/DecisionForest.h:526-533).  The kernels follow the generated code."""
    rng = np.random.Generator(np.random.PCG64(8))
    split = lambda: (rng.integers(0, 5), rng.normal())
    trees = [synth._grow_tree(rng, 4, lambda d, s: 0.9, split, lambda: rng.normal(0.0, 0.3)) for _ in range(30)]
    info = [int(c) for c in rng.choice([0, 2, 3, 5], size=len(trees))]
    path = tmp_path / "gaps.json"
    synth.write_xgboost_json(path, trees, 5, objective="multi:softmax", num_class=7, tree_info=info)
    forest = model_io.load_xgboost_json(path)
    rows = 600
    x = rng.normal(size=(rows, 5)).astype(np.float32)
    runner = make_runner(path, rows)
    if kernel == "rows_lds":
        runner.set_plan(64, 2, 2, 4096, 3)
    elif kernel == "rows_lds_one_slice":
        runner.set_plan(64, 2, 2, 4096, 1)      # one tree slice: the walk kernel keeps the arg-max itself
    elif kernel == "tree_parallel":
        runner.set_tree_parallel_plan(4, 16, 2, 0, 2)
    else:
        runner.set_global_walk_plan(128, 2, 4)
    assert "kernel=" + kernel.replace("_one_slice", "") in runner.describe_plan()
    np.testing.assert_array_equal(gpu_leaf_ids(runner, x), cpu_oracle.leaf_ids(forest, x))
    _, sums = cpu_oracle.predict(forest, x)
    voted = np.isin(np.arange(7), info)
    expected = np.where(voted[None, :], sums, forest.initial_value).astype(np.float32)
    dx = torch.from_numpy(x).cuda()
    margins = torch.zeros((rows, 7), dtype=torch.float32, device="cuda")
    classes = torch.zeros((rows,), dtype=torch.int8, device="cuda")
    torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
    runner.run_device_multiclass(dx.data_ptr(), rows, classes.data_ptr(), margins.data_ptr(), None)
    np.testing.assert_allclose(margins.cpu().numpy(), expected, rtol=RTOL_SUM, atol=1e-7)
    np.testing.assert_array_equal(classes.cpu().numpy(), cpu_oracle.argmax_generated(expected))
    np.testing.assert_array_equal(gpu_predict(runner, x), cpu_oracle.argmax_generated(expected))   # class ids only


@pytest.mark.parametrize("slices,tile_size", [(1, 1), (3, 1), (1, 2), (1, 4)])
def test_class_ties_go_to_the_larger_class_id(tmp_path, slices, tile_size):
    """Exact ties between class sums: the generated code replaces the running maximum unless it is strictly
    greater (src/reduction/LowerReduceOps.cpp:148-187), so the larger class id wins - in the finalize kernel
    and in the walk kernels' own arg-max (one tree slice)."""
    rng = np.random.Generator(np.random.PCG64(21))
    split = lambda: (rng.integers(0, 4), rng.normal())
    base = [synth._grow_tree(rng, 3, lambda d, s: 0.9, split, lambda: float(rng.integers(-2, 3)) * 0.25) for _ in range(6)]
    trees, info = [], []
    for c in (1, 3, 4):                  # three classes get the same trees: their sums tie on every row
        trees += base
        info += [c] * len(base)
    trees.append(base[0]); info.append(0)
    path = tmp_path / "ties.json"
    synth.write_xgboost_json(path, trees, 4, objective="multi:softmax", num_class=6, tree_info=info)
    forest = model_io.load_xgboost_json(path)
    rows = 900
    x = rng.normal(size=(rows, 4)).astype(np.float32)
    runner = make_tiled_runner(path, rows, tile_size, multiclass=True)
    runner.set_plan(64, 2, 2, 4096, slices)
    _, sums = cpu_oracle.predict(forest, x)
    voted = np.isin(np.arange(6), info)
    margins = np.where(voted[None, :], sums, forest.initial_value).astype(np.float32)
    expected = cpu_oracle.argmax_generated(margins)
    assert (margins[:, 1] == margins[:, 3]).all() and (margins[:, 3] == margins[:, 4]).all()
    assert set(np.unique(expected)) >= {4}            # the tie is the maximum on some rows and then class 4 wins
    np.testing.assert_array_equal(gpu_predict(runner, x), expected)


@pytest.mark.parametrize("fine", [False, True], ids=["coarse_thresholds", "fine_thresholds"])
@pytest.mark.parametrize("features", [1, 2, 63, 130, 257, 600, 1100, 3000, 4500])
@pytest.mark.parametrize("rows", [200, 3000])
def test_automatic_plan_over_feature_counts(tmp_path, features, rows, fine):
    """Whatever kernel the tuner picks for a row width (f32 tile, rank tile, tree-parallel), the answer is the oracle's."""
    rng = np.random.Generator(np.random.PCG64(features * 7 + rows + fine))
    grid = np.round(rng.normal(size=(30, features)), 2).astype(np.float32)

    def split():
        f = int(rng.integers(0, features))
        if fine and f == 0:
            return f, rng.normal()                      # feature 0 collects more than 254 distinct thresholds
        return f, grid[rng.integers(0, 30), f]
    trees = []
    for t in range(300 if fine else 60):
        tree = synth._grow_tree(rng, 6, lambda d, s: 0.85, split, lambda: rng.normal(0.0, 0.2))
        if fine:
            tree.feature[0], tree.value[0] = 0, float(np.float32(rng.normal()))
        trees.append(tree)
    path = tmp_path / "m.json"
    synth.write_xgboost_json(path, trees, features)
    forest = model_io.load_xgboost_json(path)
    x = np.round(rng.normal(size=(rows, features)), 2).astype(np.float32)
    runner = make_runner(path, rows)
    plan = runner.describe_plan()
    if features in (600, 1100) and rows > 128:            # 64 f32 rows do not fit LDS, 64 rank rows do
        assert ("quantizedRows=1" in plan) == (not fine), plan
    if features >= 3000:                                    # not even rank rows fit: a few f32 rows per block
        assert "kernel=tree_parallel" in plan, plan
    check_against_oracle(runner, forest, x)


def test_multiclass_return_type_follows_the_options(synth_model, tmp_path):
    """Default options (32-bit float results) return the class id as float32, the reference's multiclass
    setting (returnTypeWidth 8, not float) as int8; through the host-buffer entry point as well, and a
    compiled-model file keeps the choice."""
    rows = 700
    forest = model_io.load_xgboost_json(synth_model(3))
    x = synth.CONFIGS[3].batch_rows(rows, seed_offset=8)
    expected, _ = cpu_oracle.predict(forest, x)
    as_float = make_runner(synth_model(3), rows, float_class_ids=True)
    dx = torch.from_numpy(x).cuda()
    out = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()      # the library does not wait for other streams: buffers must be ready
    as_float.run_device(dx.data_ptr(), out.data_ptr(), rows)
    np.testing.assert_array_equal(out.cpu().numpy(), expected)
    np.testing.assert_array_equal(as_float.RunInference(x, np.float32), expected)
    as_int8 = make_runner(synth_model(3), rows)
    np.testing.assert_array_equal(as_int8.RunInference(x, np.int8), expected.astype(np.int8))
    for runner, dtype in ((as_float, np.float32), (as_int8, np.int8)):
        path = str(tmp_path / ("m_%s.tbamd" % np.dtype(dtype).name))
        runner.save_compiled_model(path)
        reopened = treebeard.TreebeardInferenceRunner.FromCompiledModelFile(path)
        np.testing.assert_array_equal(reopened.RunInference(x, dtype), expected.astype(dtype))
    options = treebeard.CompilerOptions(rows, 1)
    options.SetReturnTypeWidth(16)
    with pytest.raises(RuntimeError, match="8-bit integers or 32-bit floats"):
        treebeard.TreebeardInferenceRunner.FromModelFile(synth_model(3), "", options)


# The option sets of the reference's GPU auto-schedule tests (test/python/gpu_tests.py:260-325): batch 200,
# 20 rows per thread block, with and without unrolling / interleaving / tree threads, under each of its
# three GPU representation names, fed in fixed batches and compared with the model's golden CSV
# (test/python/test_utils.py:140-166).
REFERENCE_AUTO_SCHEDULES = {
    "no-cache": dict(rows_per_thread=2, unroll=False, tree_threads=1, interleave=0),
    "no-cache-unroll": dict(rows_per_thread=2, unroll=True, tree_threads=1, interleave=0),
    "unroll-treepar": dict(rows_per_thread=2, unroll=True, tree_threads=4, interleave=0),
    "unroll-interleave-treepar": dict(rows_per_thread=1, unroll=True, tree_threads=4, interleave=2),
}


@pytest.mark.parametrize("representation", ["gpu_array", "gpu_sparse", "gpu_reorg"])
@pytest.mark.parametrize("schedule", sorted(REFERENCE_AUTO_SCHEDULES))
@pytest.mark.parametrize("name", BENCHMARK_XGB)
def test_reference_auto_schedule_matrix(name, schedule, representation, plain_file):
    cfg = REFERENCE_AUTO_SCHEDULES[schedule]
    x, expected = model_io.read_csv(benchmark_csv(name))
    x = x.astype(np.float32)
    gpu = treebeard.GPUAutoScheduleOptions()
    gpu.NumberOfRowsPerThreadBlock(20)
    gpu.NumberOfRowsPerThread(cfg["rows_per_thread"])
    gpu.UnrollTreeWalks(cfg["unroll"])
    gpu.CacheRows(False)
    gpu.CacheTrees(False)
    gpu.NumberOfTreeThreads(cfg["tree_threads"])
    gpu.NumberOfTreesAtATime(1)
    if cfg["interleave"]:
        gpu.TreeWalkInterleaveFactor(cfg["interleave"])
    batch = 100                                           # the fixture CSVs hold 200 rows: two batches
    ctx = treebeard.TreebeardContext(plain_file(benchmark_model(name)), "", treebeard.CompilerOptions(batch, 1),
                                     gpuAutoScheduleOptions=gpu)
    ctx.SetRepresentationType(representation)
    ctx.SetInputFiletype("xgboost_json")
    runner = treebeard.TreebeardInferenceRunner.GPUInferenceRunnerFromTBContext(ctx)
    for first in range(0, x.shape[0], batch):
        got = runner.RunInference(x[first:first + batch], np.float32)
        np.testing.assert_allclose(got, expected[first:first + batch], rtol=RTOL_SUM, atol=ATOL_PROB)


@pytest.mark.parametrize("k,batch,rows", [(1, 256, 1000), (2, 4096, 4096 * 2 + 77), (3, 1000, 2999), (2, 1 << 18, (1 << 18) + 5),
                                          (1, 64, 64 * 5000 + 3), (4, 512, 512 * 70)])
def test_host_entry_point_takes_any_number_of_rows(synth_model, k, batch, rows):
    """The reference fixes the batch at compile time; tbmi_run_host walks longer (or shorter) host inputs in
    batch-sized windows and must give the bits of one device-resident launch."""
    x = synth.CONFIGS[k].batch_rows(rows, seed_offset=12)
    runner = make_runner(synth_model(k), batch)
    expected = gpu_predict(runner, x)
    np.testing.assert_array_equal(runner.run_host(x), expected)
    np.testing.assert_array_equal(runner.run_host(x[:batch // 3]), expected[:batch // 3])
    assert runner.run_host(x[:0]).shape == (0,)
    whole = rows // batch * batch
    np.testing.assert_array_equal(runner.RunInferenceOnMultipleBatches(x[:whole], runner.result_dtype()), expected[:whole])


def _random_forest_file(rng, path):
    features = int(rng.choice([1, 2, 5, 17, 40, 100, 300]))
    num_class = int(rng.choice([0, 0, 0, 3, 7]))
    depth = int(rng.integers(0, 11))
    trees_n = int(rng.choice([1, 2, 9, 40, 150]))
    split_p = float(rng.choice([0.5, 0.8, 1.0])) if depth <= 8 else 0.6
    lopsided = rng.random() < 0.3
    prob = (lambda d, s: (0.95 if s <= 0 else 0.2)) if lopsided else (lambda d, s: split_p)
    grid = np.round(rng.normal(size=(25, features)), 1).astype(np.float32)
    trees = [synth._grow_tree(rng, depth, prob, lambda: (lambda f: (f, grid[rng.integers(0, 25), f]))(int(rng.integers(0, features))),
                              lambda: rng.normal(0.0, 0.3), force_root=bool(rng.random() < 0.8)) for _ in range(trees_n)]
    objective = "multi:softmax" if num_class else str(rng.choice(["reg:squarederror", "binary:logistic"]))
    info = [int(c) for c in rng.permutation(trees_n) % num_class] if num_class else None
    synth.write_xgboost_json(path, trees, features, objective=objective, num_class=num_class, tree_info=info,
                             base_score=str(rng.choice(["5E-1", "2.5E-1", "0.7"])))
    return features


@pytest.mark.parametrize("seed", range(200))
def test_random_forests_and_plans(tmp_path, seed):
    """Differential run over random shapes: model, batch size, launch options; leaf ids and predictions vs the oracle."""
    rng = np.random.Generator(np.random.PCG64(9000 + seed))
    path = tmp_path / "m.json"
    features = _random_forest_file(rng, path)
    forest = model_io.load_xgboost_json(path)
    rows = int(rng.choice([1, 2, 33, 64, 129, 500, 2049, 9000]))
    x = np.round(rng.normal(size=(rows, features)), 1).astype(np.float32)      # many values sit on thresholds
    x[rng.random(x.shape) < 0.01] = np.inf
    x[rng.random(x.shape) < 0.01] = -np.inf
    gpu = None
    if rng.random() < 0.5:
        gpu = treebeard.GPUAutoScheduleOptions.Construct(num_rows_per_TB=int(rng.choice([8, 20, 64, 128, 256, 512])),
                                                         num_tree_threads=int(rng.choice([1, 2, 4, 10])))
        gpu.TreeWalkInterleaveFactor(int(rng.choice([1, 2, 4, 8])))
    runner = make_runner(path, rows, gpu_options=gpu)
    runner.set_group_staging(int(rng.integers(0, 3)))     # tree groups by rule, through registers, or copied directly
    check_against_oracle(runner, forest, x)
    kind = rng.integers(0, 5)
    try:
        if kind == 4:
            rb = int(rng.choice([64, 128, 256, 512]))
            runner.set_rank16_plan(rb, int(rng.choice([1, 2, 1024 // rb])), int(rng.choice([1, 2, 4, 8])), 0, int(rng.integers(0, 5)))
        elif kind == 0:
            runner.set_global_walk_plan(int(rng.choice([64, 256, 1024])), int(rng.choice([1, 2, 4, 8])), int(rng.integers(1, 50)))
        elif kind == 1:
            runner.set_quantized_plan(int(rng.choice([1, 4, 16])), int(rng.choice([1, 2, 4])), 0, int(rng.integers(1, 6)))
        elif kind == 2:
            lanes = int(rng.choice([1, 4, 16, 64, 256]))
            runner.set_tree_parallel_plan(max(1, 256 // lanes) if lanes < 256 else int(rng.choice([1, 2, 4])), lanes,
                                          int(rng.choice([1, 2, 4])), 0, int(rng.integers(0, 9)))
        else:
            rb = int(rng.choice([64, 128, 256]))
            runner.set_plan(rb, int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4, 8])), 0, int(rng.integers(0, 9)))
    except RuntimeError:
        pass                                              # a plan this model does not fit: refused, runner unchanged
    check_against_oracle(runner, forest, x)


@pytest.mark.parametrize("seed", range(120))
def test_random_forests_tiles_and_peeled_walks(tmp_path, seed):
    """The same differential run over the tiled walk (tile sizes 2 to 8, uniform and profile-driven tiling, peeled or
    not) and over the scalar walk with deferred tails (profile from a file or taken by the library from device rows)."""
    rng = np.random.Generator(np.random.PCG64(19000 + seed))
    path = tmp_path / "m.json"
    features = _random_forest_file(rng, path)
    forest = model_io.load_xgboost_json(path)
    rows = int(rng.choice([1, 33, 64, 129, 500, 2049, 6000]))
    x = np.round(rng.normal(size=(rows, features)), 1).astype(np.float32)
    x[rng.random(x.shape) < 0.01] = np.inf
    x[rng.random(x.shape) < 0.01] = -np.inf
    shifted = np.round(rng.normal(loc=-0.8, size=(700, features)), 1).astype(np.float32)     # the profiled rows: skewed walks
    profile = write_profile(tmp_path / "profile.csv", forest, cpu_oracle.leaf_ids(forest, shifted))
    multiclass = forest.num_classes > 0
    tile = int(rng.choice([1, 1, 2, 3, 4, 5, 6, 7, 8]))
    tiling = int(rng.integers(0, 3))
    peel = bool(rng.random() < 0.6)
    try:
        runner = make_tiled_runner(path, rows, tile, tiling, profile if (tiling or peel) else "", peel, multiclass)
    except RuntimeError as error:        # rows too wide for the tiled walk's row tile
        assert tile > 1 and "tile" in str(error), str(error)
        return
    check_against_oracle(runner, forest, x)
    if tile == 1 and rng.random() < 0.5:
        fresh = make_runner(path, rows)
        dx = torch.from_numpy(shifted).cuda()
        torch.cuda.synchronize()
        try:
            fresh.enable_peeled_walks(dx.data_ptr(), shifted.shape[0])
        except RuntimeError:
            pass                         # (a plan without the row-parallel kernel)
        check_against_oracle(fresh, forest, x)
    try:
        rb = int(rng.choice([64, 128, 256]))
        runner.set_plan(rb, int(rng.choice([1, 2, 4, 8])), int(rng.choice([1, 2, 4])), 0, int(rng.integers(0, 6)))
    except RuntimeError:
        pass
    check_against_oracle(runner, forest, x)


@pytest.mark.parametrize("k,rows", [(1, (1 << 29) + 3), (4, (1 << 20) + (1 << 18) + 5)])
def test_batches_past_32_bit_offsets(synth_model, k, rows):
    """Maximum sizes: batches of more than 2^31 elements (17 GB and 10 GB of rows, generated on the device), checked
    against the oracle on slices at both ends, in the middle and on either side of the rows where the element index
    passes 2^31 and the byte offset 2^32."""
    forest = model_io.load_xgboost_json(synth_model(k))
    features = forest.num_features
    generator = torch.Generator(device="cuda")
    generator.manual_seed(40 + k)
    x = torch.empty((rows, features), dtype=torch.float32, device="cuda")
    for lo in range(0, rows, 1 << 22):
        x[lo:lo + (1 << 22)].normal_(generator=generator)
    runner = make_runner(synth_model(k), rows)
    out = torch.zeros(rows, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    runner.run_device(x.data_ptr(), out.data_ptr(), rows)
    torch.cuda.synchronize()
    marks = [150, rows // 2, rows - 150, (1 << 31) // features, (1 << 30) // features]
    for mark in marks:
        if mark + 150 > rows:
            continue
        rows_here = x[mark - 150:mark + 150].cpu().numpy()
        pred, _ = cpu_oracle.predict(forest, rows_here)
        np.testing.assert_allclose(out[mark - 150:mark + 150].cpu().numpy(), pred, rtol=RTOL_SUM, atol=0)
    del x, out
    torch.cuda.empty_cache()


def test_lds_micro_benchmark_reports_plausible_rates():
    """The bench-only library (libtbamd_bench.so, not part of the runtime library) that bench.py quotes."""
    from treebeard_amd.runtime_api import lds_read_bandwidth
    rates = {width: lds_read_bandwidth(width) for width in (4, 8, 16)}
    assert 1e13 < rates[4] < rates[8] <= 1.3 * rates[16] < 4e14          # tens to hundreds of TB/s on 256 CUs
    with pytest.raises(RuntimeError):
        lds_read_bandwidth(3)
    from treebeard_amd.runtime_api import LDS_READ_OPS, lds_read_cost
    b32, b64 = LDS_READ_OPS.index("ds_read_b32"), LDS_READ_OPS.index("ds_read_b64")
    linear, scattered = lds_read_cost(b64, 0, 0), lds_read_cost(b64, 1, 0)
    assert 1.0 < linear < 6.0 and linear < scattered < 30.0                # bank conflicts cost cycles
    assert abs(lds_read_cost(b32, 0, 0) - linear) < 1.0                    # 4 and 8 bytes per lane cost the same
    with pytest.raises(RuntimeError):
        lds_read_cost(b32, 3, 0)


@pytest.mark.parametrize("k,rows", [(2, 20000), (3, 9000), (1, 777)])
def test_async_entry_point_orders_itself_on_the_callers_stream(synth_model, k, rows):
    """tbmi_run_device_async enqueues on the stream it is handed: inputs produced by work queued on that
    stream just before the call are seen, results are visible to work queued just after it, and no
    synchronisation is made on either side (default stream and a side stream)."""
    forest = model_io.load_xgboost_json(synth_model(k))
    x = synth.CONFIGS[k].batch_rows(rows, seed_offset=5)
    runner = make_runner(synth_model(k), rows)
    expected = gpu_predict(runner, x)
    host = torch.from_numpy(x).pin_memory()
    for stream in (torch.cuda.current_stream(), torch.cuda.Stream()):
        with torch.cuda.stream(stream):
            dx = torch.empty((rows, x.shape[1]), dtype=torch.float32, device="cuda")
            out = torch.empty((rows,), dtype=torch.int8 if runner.result_dtype() == np.int8 else torch.float32, device="cuda")
            for _ in range(3):   # keep the stream busy so that the copy below is still pending at the call
                dx.normal_()
            dx.copy_(host, non_blocking=True)
            runner.run_device_async(dx.data_ptr(), out.data_ptr(), rows, stream.cuda_stream)
            got = out.to("cpu", non_blocking=False)
        stream.synchronize()
        np.testing.assert_array_equal(got.numpy(), expected)
    pred, _ = cpu_oracle.predict(forest, x)
    if forest.num_classes == 0:
        np.testing.assert_allclose(expected, pred, rtol=RTOL_SUM, atol=ATOL_PROB)


# --------------------------------------------------------------------------
# tiled walks (CompilerOptions tile size 2 to 8) and probability-based tiling
# --------------------------------------------------------------------------
def make_tiled_runner(path, batch, tile_size, tiling_type=0, profile="", peel=False, multiclass=False):
    options = treebeard.CompilerOptions(batch, tile_size)
    options.SetTilingType(tiling_type)
    if profile:
        options.SetStatsProfileCSVPath(str(profile))
    if multiclass:
        options.SetReturnTypeWidth(8)
        options.SetReturnTypeIsFloatType(False)
    treebeard.SetPeeledCodeGenForProbabilityBasedTiling(peel)
    try:
        return treebeard.TreebeardInferenceRunner.FromModelFile(str(path), "", options)
    finally:
        treebeard.SetPeeledCodeGenForProbabilityBasedTiling(False)


def write_profile(path, forest, ids):
    """Leaf hit counts of a batch in the reference's profile format (src/utils/StatsUtils.cpp:10-52)."""
    lines = ["%d, %d" % (forest.num_trees, ids.shape[0])]
    for t in range(forest.num_trees):
        _, _, left, _ = forest.tree(t)
        counts = np.bincount(ids[:, t], minlength=len(left))
        lines.append(", ".join("%d, 0" % counts[leaf] for leaf in np.nonzero(left == -1)[0]))
    with open(path, "w") as fh:
        fh.write("\n".join(lines) + "\n")
    return str(path)


@pytest.mark.parametrize("tile_size", [2, 3, 4, 5, 7, 8])
@pytest.mark.parametrize("k,rows", [(1, 1024), (2, 4096), (3, 4096), (5, 2048)])
def test_tiled_walk_selects_the_scalar_walks_leaves(synth_model, k, rows, tile_size):
    """Set_tileSize > 1 runs the tiled kernel; its leaves are those of the scalar oracle and of the tiled CPU walk."""
    forest = model_io.load_xgboost_json(synth_model(k))
    x = synth.CONFIGS[k].batch_rows(rows, seed_offset=4)
    runner = make_tiled_runner(synth_model(k), rows, tile_size, multiclass=k == 3)
    assert " tileSize=%d " % tile_size in runner.describe_plan()
    ids = gpu_leaf_ids(runner, x)
    np.testing.assert_array_equal(ids, cpu_oracle.leaf_ids(forest, x))
    np.testing.assert_array_equal(ids, cpu_oracle.TiledForest(forest, tile_size).leaf_ids(x))
    check_against_oracle(runner, forest, x)


@pytest.mark.parametrize("tile_size", [2, 4, 8])
def test_tiled_walk_on_the_reference_fixtures(plain_file, tile_size):
    for name in BENCHMARK_XGB:
        path = plain_file(benchmark_model(name))
        data = np.loadtxt(benchmark_csv(name), delimiter=",", dtype=np.float64)
        x, expected = data[:, :-1].astype(np.float32), data[:, -1]
        forest = model_io.load_xgboost_json(path)
        runner = make_tiled_runner(path, x.shape[0], tile_size)
        np.testing.assert_array_equal(gpu_leaf_ids(runner, x), cpu_oracle.leaf_ids(forest, x))
        np.testing.assert_allclose(gpu_predict(runner, x), expected, rtol=RTOL_SUM, atol=ATOL_PROB)
    for path in random_models()[::4]:
        forest = model_io.load_xgboost_json(path)
        x = np.random.default_rng(tile_size).random((777, forest.num_features), dtype=np.float32)
        runner = make_tiled_runner(path, 777, tile_size)
        np.testing.assert_array_equal(gpu_leaf_ids(runner, x), cpu_oracle.leaf_ids(forest, x))
        np.testing.assert_array_equal(gpu_leaf_ids(runner, x), cpu_oracle.TiledForest(forest, tile_size).leaf_ids(x))


@pytest.mark.parametrize("plan", [(64, 1, 1, 16384, 1), (128, 8, 2, 32768, 3), (256, 4, 4, 40960, 2), (64, 16, 2, 24576, 5)])
@pytest.mark.parametrize("tile_size", [2, 3, 4, 6, 8])
def test_tiled_launch_plans_agree(synth_model, tile_size, plan):
    forest = model_io.load_xgboost_json(synth_model(2))
    x = synth.CONFIGS[2].batch_rows(1501, seed_offset=6)
    x[3, :] = np.inf
    x[4, :] = -np.inf
    x[5, :] = np.nan
    runner = make_tiled_runner(synth_model(2), 1501, tile_size)
    if tile_size > 4 and plan[3] < 24576:        # the biggest tree of this model takes 18 KB in 64-byte tiles
        plan = (128, 2, 1, 32768, 1)
    runner.set_plan(*plan)
    assert " tileSize=%d " % tile_size in runner.describe_plan()
    check_against_oracle(runner, forest, x)


def test_tile_sizes_the_kernels_do_not_walk_are_refused(synth_model):
    with pytest.raises(RuntimeError, match="tile size 9 is not supported"):
        make_tiled_runner(synth_model(1), 64, 9)         # the reference's own look-up table stops at 8 (256 outcomes per shape)
    with pytest.raises(RuntimeError, match="row tile below 64 KB"):
        make_tiled_runner(synth_model(4), 64, 2)          # 2000 features: no tiled row tile
    runner = make_tiled_runner(synth_model(1), 64, 2)
    with pytest.raises(RuntimeError, match="row-parallel kernel"):
        runner.set_tree_parallel_plan(4, 64, 1, 0, 1)


@pytest.mark.parametrize("tile_size,tiling_type,peel", [(4, 1, True), (4, 2, False), (2, 1, True), (3, 2, True), (1, 1, True)])
def test_profiled_runner_selects_the_same_leaves(synth_model, plain_file, tmp_path, tile_size, tiling_type, peel):
    """Probability-based / hybrid tiling and peeled walks change the layout and the trip counts, never the leaf: a
    profiled and an unprofiled runner agree on configuration 5 (skewed) and on the reference's higgs profile."""
    forest = model_io.load_xgboost_json(synth_model(5))
    x = synth.CONFIGS[5].batch_rows(3000, seed_offset=8)
    profile = write_profile(tmp_path / "c5.profile.csv", forest, cpu_oracle.leaf_ids(forest, synth.CONFIGS[5].batch_rows(4000)))
    plain = make_tiled_runner(synth_model(5), 3000, tile_size)
    profiled = make_tiled_runner(synth_model(5), 3000, tile_size, tiling_type, profile, peel)
    plan = profiled.describe_plan()
    assert " tiling=%d " % tiling_type in plan and " peelWalks=%d " % int(peel) in plan
    if tile_size > 1:
        assert int(plan.split("treesTiledByProfile=")[1].split()[0]) > 0
    expected = cpu_oracle.leaf_ids(forest, x)
    np.testing.assert_array_equal(gpu_leaf_ids(profiled, x), expected)
    np.testing.assert_array_equal(gpu_leaf_ids(plain, x), expected)
    np.testing.assert_array_equal(gpu_predict(profiled, x), gpu_predict(plain, x))
    # the reference's own profile of its higgs model
    higgs = plain_file(benchmark_model("higgs"))
    higgs_profile = plain_file(os.path.join(GOLDEN, "benchmark", "higgs.test.profile.csv.gz"))
    data = np.loadtxt(benchmark_csv("higgs"), delimiter=",", dtype=np.float64)
    hx = data[:, :-1].astype(np.float32)
    hforest = model_io.load_xgboost_json(higgs)
    runner = make_tiled_runner(higgs, hx.shape[0], tile_size, tiling_type, higgs_profile, peel)
    np.testing.assert_array_equal(gpu_leaf_ids(runner, hx), cpu_oracle.leaf_ids(hforest, hx))
    np.testing.assert_allclose(gpu_predict(runner, hx), data[:, -1], rtol=RTOL_SUM, atol=ATOL_PROB)


def test_describe_plan_says_where_walk_peeling_applies(synth_model, tmp_path):
    """Peeled walks exist for the tiled kernel and, as deferred tails, for the scalar row-parallel kernel on models
    without classes; elsewhere every bundle walks its full depth, and the plan description says so."""
    forest = model_io.load_xgboost_json(synth_model(3))
    x = synth.CONFIGS[3].batch_rows(1000, seed_offset=3)
    profile = write_profile(tmp_path / "c3.profile.csv", forest, cpu_oracle.leaf_ids(forest, synth.CONFIGS[3].batch_rows(2000)))
    runner = make_tiled_runner(synth_model(3), 1 << 17, 1, 1, profile, True, multiclass=True)
    assert " peelWalks=ignored(classes) " in runner.describe_plan()
    check_against_oracle(runner, forest, x)
    runner.set_tree_parallel_plan(4, 64, 1, 0, 1)
    assert " peelWalks=ignored(tree_parallel) " in runner.describe_plan()
    tiled = make_tiled_runner(synth_model(3), 1000, 4, 1, profile, True, multiclass=True)
    assert " peelWalks=1 " in tiled.describe_plan()
    check_against_oracle(tiled, forest, x)
    with pytest.raises(RuntimeError, match="row-parallel"):
        tiled.set_global_walk_plan(256, 4, 1)         # a tiled runner does not quietly become a scalar walk
    forest5 = model_io.load_xgboost_json(synth_model(5))
    profile5 = write_profile(tmp_path / "c5.profile.csv", forest5, cpu_oracle.leaf_ids(forest5, synth.CONFIGS[5].batch_rows(2000)))
    scalar = make_tiled_runner(synth_model(5), 4000, 1, 1, profile5, True)
    assert " peelWalks=1 " in scalar.describe_plan() and int(scalar.describe_plan().split("treesDeferred=")[1].split()[0]) > 100
    scalar.set_rank16_plan(128, 8, 4, 0, 1)
    assert " peelWalks=ignored(ranks) " in scalar.describe_plan()


@pytest.mark.parametrize("plan", [None, (256, 4, 4, 0, 1), (128, 8, 2, 24576, 3), (64, 4, 8, 16384, 7), (512, 2, 1, 32768, 1), (64, 16, 4, 0, 1)])
@pytest.mark.parametrize("k", [2, 5])
def test_deferred_tails_select_the_same_leaves(synth_model, tmp_path, k, plan):
    """Peeled walks of the scalar kernel: trees whose walks stop at a profiled level, the rows that stand on a stub
    queued per wave and walked on densely through the tail array in global memory.  Leaf ids bit-exact and the
    predictions those of an unprofiled runner, for several block shapes and tree slices, with the profile taken
    from other rows than the batch, +-inf and NaN rows, a batch that ends inside a row block, every entry point."""
    forest = model_io.load_xgboost_json(synth_model(k))
    rows = 5000 + 37
    x = synth.CONFIGS[k].batch_rows(rows, seed_offset=8)
    x[3, :] = np.inf
    x[4, :] = -np.inf
    x[5, ::3] = np.nan
    profile = write_profile(tmp_path / "profile.csv", forest, cpu_oracle.leaf_ids(forest, synth.CONFIGS[k].batch_rows(3000)))
    plain = make_tiled_runner(synth_model(k), rows, 1)
    runner = make_tiled_runner(synth_model(k), rows, 1, 1, profile, True)
    if plan and plan[0] * (forest.num_features + 1) * 4 > 150 * 1024:
        with pytest.raises(RuntimeError, match="exceeds the LDS"):
            runner.set_plan(*plan)
        return
    if plan:
        runner.set_plan(*plan)
    described = runner.describe_plan()
    if " peelWalks=1 " in described:
        assert int(described.split("treesDeferred=")[1].split()[0]) > 100, described
    else:       # a shape without room for the form says so and walks every tree to its leaves (wide row tiles, small tree groups)
        assert plan and (" peelWalks=ignored(words) " in described or " peelWalks=ignored(lds) " in described), described
    check_against_oracle(runner, forest, x)
    expected = gpu_predict(plain, x)
    np.testing.assert_allclose(gpu_predict(runner, x), expected, rtol=1e-6, atol=1e-7)    # (the tails' leaf values join the sum in another order)
    np.testing.assert_allclose(runner.RunInference(x), expected, rtol=1e-6, atol=1e-7)
    dx = torch.from_numpy(x).cuda()
    got = torch.zeros(rows, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream()
    runner.run_device_noalloc(dx.data_ptr(), got.data_ptr(), rows, stream.cuda_stream)
    stream.synchronize()
    np.testing.assert_allclose(got.cpu().numpy(), expected, rtol=1e-6, atol=1e-7)
    small = gpu_predict(runner, x[:70])                  # a batch of two row blocks at most: everything leaves through the last flush
    np.testing.assert_allclose(small, expected[:70], rtol=1e-6, atol=1e-7)


def test_deferred_tails_survive_the_compiled_model_file_and_the_plan_search(synth_model, tmp_path):
    forest = model_io.load_xgboost_json(synth_model(5))
    rows = 1 << 15
    x = synth.CONFIGS[5].batch_rows(rows, seed_offset=9)
    profile = write_profile(tmp_path / "profile.csv", forest, cpu_oracle.leaf_ids(forest, x[:3000]))
    runner = make_tiled_runner(synth_model(5), rows, 1, 1, profile, True)
    path = str(tmp_path / "deferred.tbamd")
    runner.save_compiled_model(path)
    again = treebeard.TreebeardInferenceRunner.FromSOFile(path, "")
    assert again.describe_plan() == runner.describe_plan() and " peelWalks=1 " in again.describe_plan()
    check_against_oracle(again, forest, x[:4096])
    # peeled walks without a profile file: the library profiles rows on the device itself
    fresh = make_runner(synth_model(5), rows)
    dx = torch.from_numpy(x).cuda()
    torch.cuda.synchronize()
    fresh.enable_peeled_walks(dx.data_ptr(), rows)
    assert " peelWalks=1 " in fresh.describe_plan() and int(fresh.describe_plan().split("treesDeferred=")[1].split()[0]) > 100
    check_against_oracle(fresh, forest, x[:4096])
    # the plan search of a runner without a profile profiles the batch itself and may keep deferred tails; whatever
    # it keeps selects the same leaves
    tuned = make_runner(synth_model(5), rows)
    dx = torch.from_numpy(x).cuda()
    torch.cuda.synchronize()
    tuned.autotune(dx.data_ptr(), rows)
    check_against_oracle(tuned, forest, x[:4096])


@pytest.mark.parametrize("features,rows", [(20000, 300), (40000, 70)])
def test_rows_too_wide_for_lds_walk_from_global_memory(tmp_path, features, rows):
    """More features than a 16-bit byte offset inside an LDS row can address (the reference's default 16-bit
    feature index allows 32767): the tuner falls back to the global-memory walk instead of refusing the model."""
    rng = np.random.Generator(np.random.PCG64(features))
    trees = [synth._grow_tree(rng, 6, lambda d, s: 0.85, lambda: (rng.integers(0, features), rng.normal()),
                              lambda: rng.normal(0.0, 0.2)) for _ in range(40)]
    path = tmp_path / "wide.json"
    synth.write_xgboost_json(path, trees, features)
    forest = model_io.load_xgboost_json(path)
    x = rng.normal(size=(rows, features)).astype(np.float32)
    runner = make_runner(path, rows)
    assert "kernel=global_walk" in runner.describe_plan()
    check_against_oracle(runner, forest, x)


def test_time_kernels_leaves_the_outputs_of_one_run(synth_model):
    """Repeated launches inside tbmi_time_kernels (wide finalize of a sliced classifier included) leave the same
    results as one tbmi_run_device."""
    rows = 50
    x = synth.CONFIGS[3].batch_rows(rows, seed_offset=2)
    runner = make_runner(synth_model(3), rows)
    runner.set_plan(64, 2, 2, 8192, 24)
    assert "treeSlices=24" in runner.describe_plan()
    expected = gpu_predict(runner, x)
    dx = torch.from_numpy(x).cuda()
    out = torch.full((rows,), -1, dtype=torch.int8, device="cuda")
    torch.cuda.synchronize()
    runner.time_kernels(dx.data_ptr(), out.data_ptr(), rows, 3)
    np.testing.assert_array_equal(out.cpu().numpy(), expected)

"""The entry point that allocates nothing (tbmi_run_device_noalloc) against tbmi_run_device, through the C ABI:
bit-equal results on two calls in a row, the second with a smaller input, for plans whose kernels use scratch
memory (classifier partial sums, tree slices, rank-quantised rows) and for one that uses none - and both
against the CPU oracle on the same rows."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

from oracle import cpu_oracle, model_io  # noqa: E402
from treebeard_amd import synth, treebeard  # noqa: E402
from treebeard_amd.runtime_api import api  # noqa: E402


def _runner(path, batch, multiclass):
    options = treebeard.CompilerOptions(batch, 1)
    if multiclass:
        options.SetReturnTypeWidth(8)
        options.SetReturnTypeIsFloatType(False)
    return treebeard.TreebeardInferenceRunner.FromModelFile(path, "", options)


def _both(runner, x):
    rows = x.shape[0]
    dtype = torch.int8 if runner.result_dtype() == np.int8 else torch.float32
    dx = torch.from_numpy(x).cuda()
    want = torch.zeros((rows,), dtype=dtype, device="cuda")
    got = torch.full((rows,), 77, dtype=dtype, device="cuda")
    torch.cuda.synchronize()
    runner.run_device(dx.data_ptr(), want.data_ptr(), rows)
    stream = torch.cuda.current_stream()
    runner.run_device_noalloc(dx.data_ptr(), got.data_ptr(), rows, stream.cuda_stream)
    stream.synchronize()
    return got.cpu().numpy(), want.cpu().numpy()


# (configuration, plan, rows of the first call, rows of the second call)
CASES = [
    (3, None, 6000, 1111),                       # classifier, one tree slice: arg-max kept by the walk kernel
    (3, ("plan", 256, 4, 4, 0, 2), 6000, 1111),  # classifier over two tree slices: per-class partial sums + finalize
    (2, ("plan", 256, 4, 4, 16384, 6), 3000, 500),   # tree slices: partial sums per slice
    (2, None, 70000, 4097),                      # fused epilogue: no scratch memory at all
    (4, None, 1024, 300),                        # rank-quantised rows (+ tree slices at this size)
    (1, ("tree_parallel", 4, 64, 1, 0, 3), 100, 37),
]


@pytest.mark.parametrize("k,plan,first,second", CASES)
def test_no_alloc_entry_point_matches_run_device(synth_model, k, plan, first, second):
    runner = _runner(synth_model(k), first, k == 3)
    if plan and plan[0] == "plan":
        runner.set_plan(*plan[1:])
    elif plan:
        runner.set_tree_parallel_plan(*plan[1:])
    forest = model_io.load_xgboost_json(synth_model(k))
    for call, rows in enumerate((first, second)):
        x = synth.CONFIGS[k].batch_rows(rows, seed_offset=11 + call)
        got, want = _both(runner, x)
        np.testing.assert_array_equal(got, want)
        pred, _ = cpu_oracle.predict(forest, x)         # the oracle itself, not only the allocating entry point
        if forest.num_classes > 0:
            np.testing.assert_array_equal(got.astype(np.float32), pred)
        elif forest.transform == model_io.SIGMOID:
            np.testing.assert_allclose(got, pred, rtol=0, atol=1e-6)
        else:
            np.testing.assert_allclose(got, pred, rtol=1e-5, atol=0)


def test_no_alloc_entry_point_rejects_what_does_not_fit(synth_model):
    limit = api().runtime_lib.tbmi_noalloc_scratch_bytes()
    assert limit == 32 << 20
    rows = limit // (2 * 8 * 8) + 1              # configuration 3 over two tree slices: 2 x 8 classes x 8 bytes per row
    runner = _runner(synth_model(3), rows, True)
    runner.set_plan(256, 4, 4, 0, 2)             # (with one slice the walk keeps the arg-max itself and needs no scratch)
    dx = torch.zeros((rows, 54), dtype=torch.float32, device="cuda")
    out = torch.zeros((rows,), dtype=torch.int8, device="cuda")
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="scratch memory"):
        runner.run_device_noalloc(dx.data_ptr(), out.data_ptr(), rows, None)
    runner.run_device_noalloc(dx.data_ptr(), out.data_ptr(), rows - 1, None)   # the largest call that fits
    torch.cuda.synchronize()
    want = torch.zeros((rows - 1,), dtype=torch.int8, device="cuda")
    runner.run_device(dx.data_ptr(), want.data_ptr(), rows - 1)
    np.testing.assert_array_equal(out[:rows - 1].cpu().numpy(), want.cpu().numpy())


@pytest.mark.parametrize("k,plan,rows", [(2, ("plan", 256, 4, 4, 16384, 6), 5000), (3, None, 9000), (3, ("plan", 256, 4, 4, 0, 2), 3000),
                                         (4, None, 2000)])
def test_no_alloc_entry_point_under_graph_capture(synth_model, k, plan, rows):
    """What the entry point is for: recorded into a HIP graph (no allocation, no synchronisation, no memset on its
    path) and replayed several times on new input, with eager work and synchronisations between the replays; every
    replay gives what an eager call gives, and what the oracle gives."""
    runner = _runner(synth_model(k), rows, k == 3)
    if plan:
        runner.set_plan(*plan[1:])
    forest = model_io.load_xgboost_json(synth_model(k))
    dtype = torch.int8 if runner.result_dtype() == np.int8 else torch.float32
    fixed_in = torch.zeros((rows, forest.num_features), dtype=torch.float32, device="cuda")
    fixed_out = torch.zeros((rows,), dtype=dtype, device="cuda")
    eager = torch.zeros_like(fixed_out)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):       # an eager call first: kernel attributes are set at a kernel's first launch
        runner.run_device_noalloc(fixed_in.data_ptr(), fixed_out.data_ptr(), rows, side.cuda_stream)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        runner.run_device_noalloc(fixed_in.data_ptr(), fixed_out.data_ptr(), rows, torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        x = synth.CONFIGS[k].batch_rows(rows, seed_offset=30 + replay)
        fixed_in.copy_(torch.from_numpy(x))
        fixed_out.fill_(77)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        runner.run_device(fixed_in.data_ptr(), eager.data_ptr(), rows)
        np.testing.assert_array_equal(fixed_out.cpu().numpy(), eager.cpu().numpy())
        pred, _ = cpu_oracle.predict(forest, x)
        if k == 3:
            np.testing.assert_array_equal(fixed_out.cpu().numpy().astype(np.float32), pred.astype(np.float32))
        else:
            np.testing.assert_allclose(fixed_out.cpu().numpy(), pred, rtol=1e-5, atol=1e-6)

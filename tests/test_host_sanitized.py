"""The host side of the library compiled with sanitizers, no GPU and no HIP runtime involved.

test_host_code_under_sanitizers: loaders, packer, tuner, compiled-model file and the pinned-staging copier
under AddressSanitizer + UndefinedBehaviorSanitizer over the five configurations with every launch-plan shape
the GPU tests pin.

test_runner_under_*: the runner and the whole C ABI (runner.cpp, runtime.cpp) linked against a host-only
stand-in for the HIP runtime whose "kernels" interpret the packed model on the CPU (tests/native/
hip_host_shim.cpp), driven through host and device entry points of many sizes, plan changes, the plan search
and the compiled-model file: every buffer the runner sizes and every copy it makes is seen by ASan/UBSan, the
copier threads by ThreadSanitizer."""
import concurrent.futures
import os
import shutil
import subprocess

import pytest

from treebeard_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "treebeard_amd", "csrc")
HOST_SOURCES = ["forest.cpp", "json_reader.cpp", "xgboost_loader.cpp", "packer.cpp", "tuner.cpp", "model_file.cpp", "host_copy.cpp"]


def _compile_and_link(tmp_path, flags, sources, exe):
    """One g++ per source file, four at a time, then the link: the sanitizer builds are most of these tests' time."""
    def compile_one(source):
        obj = str(tmp_path / (os.path.basename(source) + "." + os.path.basename(exe) + ".o"))
        return obj, subprocess.run(["g++"] + flags + ["-c", source, "-o", obj], capture_output=True, text=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(compile_one, sources))
    for _, built in results:
        if built.returncode != 0:
            return built
    sanitize = [f for f in flags if f.startswith("-fsanitize=")]
    return subprocess.run(["g++"] + sanitize + [obj for obj, _ in results] + ["-lpthread", "-o", exe], capture_output=True, text=True)


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_host_code_under_sanitizers(tmp_path, synth_model, host_driver):
    exe = host_driver
    models = [synth_model(k) for k in (1, 2, 3, 4, 5)]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", TMPDIR=str(tmp_path))
    run = subprocess.run([exe] + models, capture_output=True, text=True, env=env, timeout=900)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert "ok" in run.stdout


RUNNER_SOURCES = HOST_SOURCES + ["onnx_loader.cpp", "runner.cpp", "runtime.cpp"]


def _build_runner_driver(tmp_path, sanitize):
    exe = str(tmp_path / ("sanitize_runner_" + sanitize.split(",")[0]))
    flags = ["-std=c++17", "-O1", "-g", "-fsanitize=" + sanitize, "-fno-omit-frame-pointer",
             "-D__HIP_PLATFORM_AMD__", "-D__align__(x)=__attribute__((aligned(x)))", "-DHIP_SYMBOL(x)=x",
             "-I", "/opt/rocm/include", "-I", CSRC]
    if "undefined" in sanitize:
        flags.append("-fno-sanitize-recover=undefined")
    sources = [os.path.join(HERE, "native", "sanitize_runner.cpp"), os.path.join(HERE, "native", "hip_host_shim.cpp")]
    built = _compile_and_link(tmp_path, flags, sources + [os.path.join(CSRC, s) for s in RUNNER_SOURCES], exe)
    if built.returncode != 0 and ("sanitize" in built.stderr or "hip/hip_runtime" in built.stderr):
        pytest.skip("this g++ has no sanitizer runtime, or the HIP headers are missing")
    assert built.returncode == 0, built.stderr[-3000:]
    return exe


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_loaders_survive_mutated_files(tmp_path, host_driver):
    """Flipped bytes, overwritten words, cut and doubled pieces in an XGBoost JSON file, an ONNX file and a compiled-model
    file: every mutant is refused with an error or loads into a forest that validates and packs, under ASan + UBSan."""
    import sys
    import numpy as np
    sys.path.insert(0, HERE)
    from onnx_writer import write_onnx
    rng = np.random.Generator(np.random.PCG64(11))
    trees = [synth._grow_tree(rng, 4, lambda d, s: 0.8, lambda: (rng.integers(0, 6), np.round(rng.normal(), 2)),
                              lambda: rng.normal(0.0, 0.1)) for _ in range(6)]
    json_path = str(tmp_path / "small.json")
    synth.write_xgboost_json(json_path, trees, 6, objective="binary:logistic")
    onnx_path = str(tmp_path / "small.onnx")
    write_onnx(onnx_path, [(t.value, t.feature, t.left, t.right) for t in trees], post_transform="LOGISTIC")
    exe = str(tmp_path / "mutate_loaders")
    flags = ["-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
             "-fno-omit-frame-pointer", "-I", CSRC]
    sources = [os.path.join(HERE, "native", "mutate_loaders.cpp")] + [os.path.join(CSRC, s) for s in HOST_SOURCES + ["onnx_loader.cpp"]]
    built = _compile_and_link(tmp_path, flags, sources, exe)
    if built.returncode != 0 and "sanitize" in built.stderr:
        pytest.skip("this g++ has no sanitizer runtime")
    assert built.returncode == 0, built.stderr[-2000:]
    # a compiled-model file of the same forest, written by the library's own writer (through the host-side driver)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:allocator_may_return_null=0:max_allocation_size_mb=4096",
               TMPDIR=str(tmp_path))
    run = subprocess.run([host_driver, json_path], capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0, (run.stdout + run.stderr)[-3000:]
    compiled = str(tmp_path / "sanitize_model.tbamd")
    assert os.path.exists(compiled)
    # a hit-count profile of the same forest in the reference's format (src/utils/StatsUtils.cpp:10-52)
    profile_path = str(tmp_path / "profile.csv")
    with open(profile_path, "w") as fh:
        fh.write("%d, 1000\n" % len(trees))
        for t in trees:
            leaves = [n for n in range(len(t.left)) if t.left[n] == -1]
            fh.write(", ".join("%d, 0" % rng.integers(0, 1000) for _ in leaves) + "\n")
    run = subprocess.run([exe, "600", "json", json_path, "onnx", onnx_path, "6", "compiled", compiled, "profile", profile_path, json_path],
                         capture_output=True, text=True, env=env, timeout=900)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert run.stdout.strip().endswith("ok"), run.stdout[-500:]


@pytest.fixture(scope="module")
def address_driver(tmp_path_factory):
    """The runner driver under ASan + UBSan, built once for the tests that use it."""
    return _build_runner_driver(tmp_path_factory.mktemp("address_driver"), "address,undefined")


@pytest.fixture(scope="module")
def host_driver(tmp_path_factory):
    """tests/native/sanitize_host.cpp under ASan + UBSan, built once."""
    where = tmp_path_factory.mktemp("host_driver")
    exe = str(where / "sanitize_host")
    flags = ["-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
             "-fno-omit-frame-pointer", "-I", CSRC]
    built = _compile_and_link(where, flags, [os.path.join(HERE, "native", "sanitize_host.cpp")] + [os.path.join(CSRC, s) for s in HOST_SOURCES], exe)
    if built.returncode != 0 and "sanitize" in built.stderr:
        pytest.skip("this g++ has no sanitizer runtime")
    assert built.returncode == 0, built.stderr[-2000:]
    return exe


def _wide_model(tmp_path):
    """40 trees over 600 features: 8300 rows are 20 MB of input, enough for the host entry point to send them
    in pieces through its pinned buffers, and cheap to walk on the CPU."""
    import numpy as np
    rng = np.random.Generator(np.random.PCG64(5))
    trees = [synth._grow_tree(rng, 6, lambda d, s: 0.9, lambda: (rng.integers(0, 600), rng.standard_normal()),
                              lambda: rng.normal(0.0, 0.1)) for _ in range(40)]
    path = str(tmp_path / "wide600.json")
    synth.write_xgboost_json(path, trees, 600)
    return path


def _multiclass_model(tmp_path):
    """160 complete trees of depth 6 voting for 8 classes over 54 features: the shape of the multiclass benchmark
    configuration at a fifth of its trees (every plan shape is re-packed under the sanitizers dozens of times)."""
    import numpy as np
    rng = np.random.Generator(np.random.PCG64(6))
    trees = [synth._grow_tree(rng, 6, lambda d, s: 1.0, lambda: (rng.integers(0, 54), float(np.round(rng.normal(), 2))),
                              lambda: rng.normal(0.0, 0.1)) for _ in range(160)]
    path = str(tmp_path / "multiclass160.json")
    synth.write_xgboost_json(path, trees, 54, objective="multi:softmax", num_class=8, tree_info=[t % 8 for t in range(160)])
    return path


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_runner_under_address_sanitizer(tmp_path, synth_model, address_driver):
    exe = address_driver
    args = [_wide_model(tmp_path), "8300", synth_model(4), "300", _multiclass_model(tmp_path), "300", synth_model(1), "9000"]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", TMPDIR=str(tmp_path))
    run = subprocess.run([exe] + args, capture_output=True, text=True, env=env, timeout=900)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert run.stdout.strip().endswith("ok")


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_runner_survives_mutated_compiled_models(tmp_path, synth_model, address_driver):
    """tbmi_load_compiled_model on compiled-model files whose header words (plan, batch size, return type, counts) and
    body were overwritten: refused with a message or loaded and run on a few rows, under ASan + UBSan."""
    exe = address_driver
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:max_allocation_size_mb=8192", TMPDIR=str(tmp_path))
    run = subprocess.run([exe, synth_model(1), "64"], capture_output=True, text=True, env=env, timeout=900)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    compiled = str(tmp_path / "sanitize_runner.tbamd")
    assert os.path.exists(compiled)
    run = subprocess.run([exe, "--mutate", compiled, "1500"], capture_output=True, text=True, env=env, timeout=900)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert run.stdout.strip().endswith("ok"), run.stdout[-500:]


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_runner_under_thread_sanitizer(tmp_path, synth_model):
    exe = _build_runner_driver(tmp_path, "thread")
    env = dict(os.environ, SANITIZE_QUICK="1", TMPDIR=str(tmp_path))
    run = subprocess.run([exe, _wide_model(tmp_path), "8300"], capture_output=True, text=True, env=env, timeout=900)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert run.stdout.strip().endswith("ok")

"""The host side of the library (loaders, packer, tuner, compiled-model file, the pinned-staging copier)
compiled with AddressSanitizer + UndefinedBehaviorSanitizer and driven over the five configurations with
every launch-plan shape the GPU tests pin.  No GPU and no HIP runtime involved."""
import os
import shutil
import subprocess

import pytest

from treebeard_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "treebeard_amd", "csrc")
HOST_SOURCES = ["forest.cpp", "json_reader.cpp", "xgboost_loader.cpp", "packer.cpp", "tuner.cpp", "model_file.cpp", "host_copy.cpp"]


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_host_code_under_sanitizers(tmp_path, synth_model):
    exe = str(tmp_path / "sanitize_host")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-fno-omit-frame-pointer", "-I", CSRC, os.path.join(HERE, "native", "sanitize_host.cpp")]
    cmd += [os.path.join(CSRC, s) for s in HOST_SOURCES] + ["-lpthread", "-o", exe]
    built = subprocess.run(cmd, capture_output=True, text=True)
    if built.returncode != 0 and "sanitize" in built.stderr:
        pytest.skip("this g++ has no sanitizer runtime")
    assert built.returncode == 0, built.stderr[-2000:]
    models = [synth_model(k) for k in (1, 2, 3, 4, 5)]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", TMPDIR=str(tmp_path))
    run = subprocess.run([exe] + models, capture_output=True, text=True, env=env, timeout=900)
    assert run.returncode == 0, (run.stdout + run.stderr)[-4000:]
    assert "ok" in run.stdout

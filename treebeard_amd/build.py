"""Builds the runtime library (libtreebeard_amd.so) and the bench-only micro-benchmark library
(libtbamd_bench.so) in-tree with hipcc for gfx950."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtreebeard_amd.so")
BENCH_LIB = os.path.join(HERE, "libtbamd_bench.so")
SOURCES = ["forest.cpp", "json_reader.cpp", "xgboost_loader.cpp", "onnx_loader.cpp", "packer.cpp", "tuner.cpp", "model_file.cpp",
           "host_copy.cpp", "runner.cpp", "runtime.cpp", "kernels.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose=False):
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in SOURCES:
        obj = os.path.join(HERE, "build", src.rsplit(".", 1)[0] + ".o")
        objs.append(obj)
        cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if src.endswith(".cpp"):
            cmd[1:1] = ["-x", "hip"]
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            failed = True
            sys.stderr.write("== %s failed ==\n%s\n" % (src, out))
        elif verbose and out:
            sys.stderr.write("== %s ==\n%s\n" % (src, out))
    if failed:
        raise RuntimeError("hipcc failed")
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs, check=True)
    bench = subprocess.run([HIPCC] + FLAGS + ["-shared", os.path.join(CSRC, "bench_kernels.hip"), "-o", BENCH_LIB],
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if bench.returncode != 0:
        sys.stderr.write("== bench_kernels.hip failed ==\n%s\n" % bench.stdout)
        raise RuntimeError("hipcc failed")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))

import gzip
import os
import shutil
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir():
    return GOLDEN


@pytest.fixture(scope="session")
def work_dir(tmp_path_factory):
    return str(tmp_path_factory.mktemp("tbamd"))


@pytest.fixture(scope="session")
def plain_file(work_dir):
    """Returns a function mapping a fixture path (possibly .gz) to an uncompressed file path."""
    cache = {}

    def get(path):
        path = str(path)
        if not path.endswith(".gz"):
            return path
        if path not in cache:
            out = os.path.join(work_dir, os.path.basename(path)[:-3])
            with gzip.open(path, "rb") as fi, open(out, "wb") as fo:
                shutil.copyfileobj(fi, fo)
            cache[path] = out
        return cache[path]

    return get


@pytest.fixture(scope="session")
def synth_model(work_dir):
    """Returns a function k -> path of benchmark configuration k's XGBoost-JSON model."""
    from treebeard_amd import synth

    def get(k):
        return synth.model_path(k, os.path.join(work_dir, "synth"))

    return get


def random_models():
    out = []
    for family in ("Random_1Tree", "Random_2Tree", "Random_4Tree"):
        d = os.path.join(GOLDEN, family)
        for name in sorted(os.listdir(d)):
            if name.endswith(".json"):
                out.append(os.path.join(d, name))
    return out


BENCHMARK_XGB = ["higgs", "airline", "year_prediction_msd"]


def benchmark_model(name):
    return os.path.join(GOLDEN, "benchmark", name + "_xgb_model_save.json.gz")


def benchmark_csv(name):
    return os.path.join(GOLDEN, "benchmark", name + "_xgb_model_save.json.csv")

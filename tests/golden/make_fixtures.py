"""Copies the reference's own test DATA (model files and XGBoost / ONNX golden
CSVs) into tests/golden/ so that the suite runs where the reference checkout
is absent.  Data only: model files are copied byte for byte (gzip-compressed
when large) and golden CSVs are cut to their first rows.  Run from the repo
root in a container that has /root/reference:

    python tests/golden/make_fixtures.py
"""
import gzip
import os
import shutil
import sys

REF = os.environ.get("TREEBEARD_REFERENCE", "/root/reference")
OUT = os.path.dirname(os.path.abspath(__file__))
CSV_ROWS = 200


def copy(src, dst, gz=False):
    os.makedirs(os.path.dirname(dst), exist_ok=True)
    if gz:
        with open(src, "rb") as fi, gzip.GzipFile(dst + ".gz", "wb", mtime=0) as fo:
            shutil.copyfileobj(fi, fo)
    else:
        shutil.copyfile(src, dst)


def head(src, dst, rows=CSV_ROWS):
    os.makedirs(os.path.dirname(dst), exist_ok=True)
    with open(src) as fi, open(dst, "w") as fo:
        for i, line in enumerate(fi):
            if i >= rows:
                break
            fo.write(line)


def main():
    xgb = os.path.join(REF, "xgb_models")
    onnx = os.path.join(REF, "onnx_models")
    for name in ("leftheavy", "rightheavy", "rightandleftheavy"):
        copy(os.path.join(xgb, "test", name + "_xgb_model.json"), os.path.join(OUT, "handbuilt", name + "_xgb_model.json"))
    # every fourth random model of each family (listed by the reference's ModelList.txt)
    for family in ("Random_1Tree", "Random_2Tree", "Random_4Tree"):
        with open(os.path.join(xgb, "test", family, "ModelList.txt")) as fh:
            models = [l.strip() for l in fh if l.strip()]
        for name in sorted(models)[::4]:
            copy(os.path.join(xgb, "test", family, name), os.path.join(OUT, family, name))
            head(os.path.join(xgb, "test", family, name + ".csv"), os.path.join(OUT, family, name + ".csv"))
    for name in ("higgs", "airline", "year_prediction_msd"):
        base = name + "_xgb_model_save.json"
        copy(os.path.join(xgb, base), os.path.join(OUT, "benchmark", base), gz=True)
        head(os.path.join(xgb, base + ".csv"), os.path.join(OUT, "benchmark", base + ".csv"))
    copy(os.path.join(onnx, "abalone_onnx_model_save.onnx"), os.path.join(OUT, "benchmark", "abalone_onnx_model_save.onnx"), gz=True)
    head(os.path.join(onnx, "abalone_onnx_model_save.onnx.csv"), os.path.join(OUT, "benchmark", "abalone_onnx_model_save.onnx.csv"))
    copy(os.path.join(onnx, "higgs_xgb_model_save.onnx"), os.path.join(OUT, "benchmark", "higgs_xgb_model_save.onnx"), gz=True)
    # leaf hit-count profile (src/utils/StatsUtils.cpp:10-52 format) for the probability-aware layout
    prof = os.path.join(xgb, "profiles", "higgs.test.csv")
    if os.path.exists(prof):
        copy(prof, os.path.join(OUT, "benchmark", "higgs.test.profile.csv"), gz=True)


if __name__ == "__main__":
    sys.exit(main())

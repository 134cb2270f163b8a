"""Builds libevotrees_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libevotrees_hip.so")
SOURCES = ["api.hip", "kernels_data.hip", "kernels_grad.hip", "kernels_hist.hip", "kernels_scan.hip", "kernels_part.hip",
           "kernels_predict.hip", "predict_static.hip", "kernels_quantile.hip", "probes.hip"]
# -ffp-contract=off: the split gains follow the reference's expression order without fused multiply-add.
# packed-fp32 instructions are disabled for all device code.
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wall", "-Wno-unused-result"]


def _compile(src):
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = ["hipcc"] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, res.stdout, res.stderr))
    return obj, res.stderr


def build(verbose=False):
    with ThreadPoolExecutor(max_workers=4) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [r[0] for r in results]
    if verbose:
        for _, err in results:
            if err.strip():
                sys.stderr.write(err)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (res.stdout, res.stderr))
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))

"""Builds libthundergbm.so and the two CLIs for gfx950 with hipcc (in-tree, no cmake needed)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libthundergbm.so")
CALIBRATION_LIB = os.path.join(HERE, "libtgbm_calibration.so")
BIN_DIR = os.path.join(HERE, "bin")

HIP_SOURCES = ["tree_kernels.hip", "sparse_kernels.hip", "prep_kernels.hip", "predict_kernels.hip", "rank_kernels.hip", "trainer.hip",
               "predictor.hip", "capi.hip", "predict_noalloc.hip"]
CPP_SOURCES = ["host_io.cpp"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-munsafe-fp-atomics",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-result"]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build(force=True):
    """Compiles every source. With force=False nothing is done when the library is newer than all sources."""
    srcs = [os.path.join(CSRC, f) for f in HIP_SOURCES + CPP_SOURCES]
    deps = srcs + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    if not force and os.path.exists(LIB) and all(os.path.getmtime(LIB) >= os.path.getmtime(d) for d in deps):
        return LIB
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for f in HIP_SOURCES + CPP_SOURCES:
        obj = os.path.join(HERE, "build", f.rsplit(".", 1)[0] + ".o")
        cmd = [HIPCC] + COMMON + ["-c", os.path.join(CSRC, f), "-o", obj]
        print(" ".join(cmd), flush=True)
        procs.append((subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True), f))
        objs.append(obj)
    failed = False
    for p, f in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip():
            print(out)
        if p.returncode != 0:
            failed = True
            print("FAILED:", f)
    if failed:
        raise RuntimeError("hipcc failed")
    _run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs)
    # the profiler calibration helper is a library of its own (not part of the training library's ABI)
    _run([HIPCC] + COMMON + ["-shared", os.path.join(CSRC, "calibration_copy.hip"), "-o", CALIBRATION_LIB])
    os.makedirs(BIN_DIR, exist_ok=True)
    for name, src in (("thundergbm-train", "cli_train.cpp"), ("thundergbm-predict", "cli_predict.cpp")):
        _run([HIPCC, "-O2", "-std=c++17", os.path.join(CSRC, src), "-o", os.path.join(BIN_DIR, name),
              "-L" + HERE, "-lthundergbm", "-Wl,-rpath,$ORIGIN/.."])
    return LIB


if __name__ == "__main__":
    build(force="--if-needed" not in sys.argv)

"""Build librtvla.so (gfx950) in-tree with hipcc: python build.py [-v] [-DNAME ...] [-o OUT.so]
(-D / -o make a variant build, e.g. -DRTVLA_TUNING with its environment knobs, next to the shipped library)."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librtvla.so")
SOURCES = ["gemm.hip", "gemm8.hip", "skinny.hip", "attention.hip", "misc.hip", "dm0.hip", "flash.hip", "rtvla.hip", "transforms.hip"]
# bit-exact parity with host arithmetic (Pillow, numpy): no fused multiply-adds in these files
# flash.hip: MFMA results in ordinary VGPRs (the softmax reads every logit; the accumulator-register form costs a copy each)
EXTRA = {"transforms.hip": ["-ffp-contract=off"], "flash.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"], "attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-unused-value",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc():
    for p in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if p and (os.path.sep not in p or os.path.exists(p)):
            return p
    return "hipcc"


def _compile(job):
    src, defines, tag = job
    obj = os.path.join(CSRC, src.replace(".hip", tag + ".o"))
    cmd = [_hipcc()] + FLAGS + list(defines) + EXTRA.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and "warnings generated" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    return obj, err


def build(force=True, verbose=False, defines=(), out=LIB):
    """Compile every HIP source for gfx950 and link the shared library."""
    if not force and os.path.exists(out):
        return out
    tag = "" if out == LIB else "." + os.path.splitext(os.path.basename(out))[0]
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 4)) as ex:
        results = list(ex.map(_compile, [(src, defines, tag) for src in SOURCES]))
    if verbose:
        for _, err in results:
            if err.strip():
                print(err)
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + [o for o, _ in results]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return out


if __name__ == "__main__":
    argv = sys.argv[1:]
    out = os.path.abspath(argv[argv.index("-o") + 1]) if "-o" in argv else LIB
    print(build(force=True, verbose="-v" in argv, defines=[a for a in argv if a.startswith("-D")], out=out))

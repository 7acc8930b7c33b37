"""The library's host code (context tables, binding, workspace layout, size planning, argument checks: csrc/rtvla.hip and
csrc/transforms.hip) compiled with AddressSanitizer and UndefinedBehaviorSanitizer on the host side only (device code is
left alone) and driven through the C ABI by tests/host_sanitizer_driver.cpp.  No GPU is needed: every call in the driver
returns before a device is touched.  Any sanitizer report aborts the driver (-fno-sanitize-recover)."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "realtime-vla_amd")
CSRC = os.path.join(PKG, "csrc")
sys.path.insert(0, PKG)

SANITIZED = ["rtvla.hip", "transforms.hip"]       # the files with host logic; the others hold kernels and their launchers


def _run(cmd, **kw):
    r = subprocess.run(cmd, capture_output=True, text=True, **kw)
    assert r.returncode == 0, "%s\n%s" % (" ".join(cmd), (r.stdout + r.stderr)[-4000:])
    return r


@pytest.mark.timeout(900)
def test_c_abi_host_paths_are_clean_under_asan_and_ubsan(tmp_path):
    import build as rtvla_build
    hipcc = rtvla_build._hipcc()
    if shutil.which(hipcc) is None and not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    plain = [os.path.join(CSRC, s.replace(".hip", ".o")) for s in rtvla_build.SOURCES if s not in SANITIZED]
    if not all(os.path.exists(o) for o in plain):
        rtvla_build.build(force=True)
    objs = []
    for src in SANITIZED:
        obj = str(tmp_path / src.replace(".hip", ".san.o"))
        san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host", "-fno-sanitize-recover=undefined"]
        _run([hipcc] + [f for f in rtvla_build.FLAGS if f != "-O3"] + ["-O1", "-g"] + rtvla_build.EXTRA.get(src, []) + san +
             ["-c", os.path.join(CSRC, src), "-o", obj])
        objs.append(obj)
    clangxx = "/opt/rocm/lib/llvm/bin/clang++"
    cxx = clangxx if os.path.exists(clangxx) else "g++"
    drv_o = str(tmp_path / "driver.o")
    _run([cxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-c",
          os.path.join(ROOT, "tests", "host_sanitizer_driver.cpp"), "-o", drv_o])
    exe = str(tmp_path / "host_sanitizer_driver")
    _run([hipcc, "--offload-arch=gfx950", "-fsanitize=address", "-fsanitize=undefined", "-fno-gpu-sanitize", drv_o] + objs + plain + ["-o", exe])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    r = _run([exe], env=env)
    assert "all checks passed" in r.stdout

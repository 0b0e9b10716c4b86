"""Build recipe for the native libraries (hipcc, gfx950 only).

  libkx_hip.so   HIP kernels + C ABI            (csrc/*.hip)
  libkuiper.so   C++ host API over that C ABI    (kuiper/source/**/*.cpp)
  test_kuiper    C++ test runner for the host API (kuiper/test/*.cpp)

Everything lands under mykuiperllama_amd/lib/, in-tree, so that a snapshot of the repository
carries the binaries to a machine that only runs them.
"""
import glob
import os
import subprocess

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
LIB_DIR = os.path.join(PKG, "lib")
CSRC = os.path.join(PKG, "csrc")
KUIPER = os.path.join(PKG, "kuiper")
INCLUDE = os.path.join(ROOT, "include")

KX_LIB = os.path.join(LIB_DIR, "libkx_hip.so")
KUIPER_LIB = os.path.join(LIB_DIR, "libkuiper.so")
KUIPER_TEST = os.path.join(LIB_DIR, "test_kuiper")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed fp32 VALU forms are switched off for all device code
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON = ["-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-command-line-argument"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd) + "\n" + out)
    return out


def build_kx():
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    _run([HIPCC] + DEVICE_FLAGS + COMMON + ["-shared", "-I", INCLUDE, "-I", CSRC] + srcs + ["-o", KX_LIB])
    return KX_LIB


def build_kuiper():
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(KUIPER, "source", "**", "*.cpp"), recursive=True))
    if not srcs:
        return None
    inc = ["-I", INCLUDE, "-I", os.path.join(KUIPER, "include"), "-I", os.path.join(KUIPER, "source", "op")]
    _run([HIPCC] + DEVICE_FLAGS + COMMON + ["-shared"] + inc + srcs +
         ["-L", LIB_DIR, "-lkx_hip", "-Wl,-rpath,$ORIGIN", "-o", KUIPER_LIB])
    tests = sorted(glob.glob(os.path.join(KUIPER, "test", "*.cpp")))
    if tests:
        _run([HIPCC] + DEVICE_FLAGS + COMMON + inc + ["-I", os.path.join(KUIPER, "test")] + tests +
             ["-L", LIB_DIR, "-lkuiper", "-lkx_hip", "-Wl,-rpath,$ORIGIN", "-o", KUIPER_TEST])
    return KUIPER_LIB


def build_all():
    build_kx()
    build_kuiper()


if __name__ == "__main__":
    build_all()
    print("built:", KX_LIB, KUIPER_LIB if os.path.exists(KUIPER_LIB) else "")

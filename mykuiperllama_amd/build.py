"""Build recipe for the native libraries (hipcc, gfx950 only).

  libkx_hip.so   HIP kernels + C ABI            (csrc/*.hip)
  libkuiper.so   C++ host API over that C ABI    (kuiper/source/**/*.cpp)
  test_kuiper    C++ test runner for the host API (tests/cpp/*, links oracle/kx_oracle.c)
  kx_safetensors_dump   lists the tensors of a checkpoint file (kuiper/app/safetensors_dump.cpp)
  libkx_probe.so  measurement only: the streaming-read kernel bench.py uses as the floor (probe/*.hip)
  test_kuiper_asan  optional (--asan): the host API and its C++ tests with AddressSanitizer on the host code

`python -m mykuiperllama_amd.build --ablate N` builds lib/libkx_hip_ablateN.so (only that), the HIP
library with parts of the GEMV kernels compiled out (-DKX_ABLATE=N: 1 = no split-K exchange, 2 = loads
only, 3 = loads and arithmetic but neither the reduction across lanes and waves nor the exchange, on the
vector kernel's plain launch; the other kernels as with 1; 4, 5, 6 = the first attention stage cut short: 4 = loads
only, 5 = through the softmax statistics and the arrival of the V rows, 6 = everything but the stores of the
weighted sums, the GEMV kernels whole); `bench.py --lib` times it.  Its results are wrong by construction: it exists
to attribute time.

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
TESTS_CPP = os.path.join(ROOT, "tests", "cpp")

KX_LIB = os.path.join(LIB_DIR, "libkx_hip.so")
KUIPER_LIB = os.path.join(LIB_DIR, "libkuiper.so")
KUIPER_TEST = os.path.join(LIB_DIR, "test_kuiper")
SAFETENSORS_DUMP = os.path.join(LIB_DIR, "kx_safetensors_dump")
QWEN3_DECODE = os.path.join(LIB_DIR, "kx_qwen3_decode")
PROBE_LIB = os.path.join(LIB_DIR, "libkx_probe.so")
PROBE_SRC = os.path.join(PKG, "probe")

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


def build_kx(ablate=0):
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    out = KX_LIB if not ablate else os.path.join(LIB_DIR, f"libkx_hip_ablate{int(ablate)}.so")
    defines = [f"-DKX_ABLATE={int(ablate)}"] if ablate else []
    _run([HIPCC] + DEVICE_FLAGS + COMMON + defines + ["-shared", "-I", INCLUDE, "-I", CSRC] + srcs + ["-o", out])
    return out


def build_probe():
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(PROBE_SRC, "*.hip")))
    _run([HIPCC] + DEVICE_FLAGS + COMMON + ["-shared"] + srcs + ["-o", PROBE_LIB])
    return PROBE_LIB


def build_kuiper():
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(KUIPER, "source", "**", "*.cpp"), recursive=True) +
                  glob.glob(os.path.join(KUIPER, "source", "**", "*.hip"), recursive=True))
    if not srcs:
        return None
    inc = ["-I", INCLUDE, "-I", os.path.join(KUIPER, "include"), "-I", os.path.join(KUIPER, "source", "op")]
    _run([HIPCC] + DEVICE_FLAGS + COMMON + ["-shared"] + inc + srcs +
         ["-L", LIB_DIR, "-lkx_hip", "-Wl,-rpath,$ORIGIN", "-o", KUIPER_LIB])
    _run([HIPCC, "--offload-arch=gfx950"] + COMMON + inc + [os.path.join(KUIPER, "app", "safetensors_dump.cpp")] +
         ["-L", LIB_DIR, "-lkuiper", "-lkx_hip", "-Wl,-rpath,$ORIGIN", "-o", SAFETENSORS_DUMP])
    _run([HIPCC, "--offload-arch=gfx950"] + COMMON + inc + [os.path.join(KUIPER, "app", "qwen3_decode.cpp")] +
         ["-L", LIB_DIR, "-lkuiper", "-lkx_hip", "-Wl,-rpath,$ORIGIN", "-o", QWEN3_DECODE])
    # C++ tests of the host API live under tests/cpp and link the CPU oracle as their checker
    tests = sorted(glob.glob(os.path.join(TESTS_CPP, "*.cpp")) + glob.glob(os.path.join(TESTS_CPP, "*.hip")))
    if tests:
        oracle_obj = os.path.join(LIB_DIR, "kx_oracle_for_tests.o")
        _run(["gcc", "-O2", "-fPIC", "-std=c11", "-c", os.path.join(ROOT, "oracle", "kx_oracle.c"), "-o", oracle_obj])
        objs = [oracle_obj]
        obj_dir = os.path.join(LIB_DIR, "obj")
        os.makedirs(obj_dir, exist_ok=True)
        for src in tests:  # one object per source: hipcc would read a mixed .hip/.o line as all-HIP
            obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
            _run([HIPCC] + DEVICE_FLAGS + COMMON + inc + ["-I", TESTS_CPP, "-c", src, "-o", obj])
            objs.append(obj)
        _run([HIPCC, "--offload-arch=gfx950"] + objs +
             ["-L", LIB_DIR, "-lkuiper", "-lkx_hip", "-Wl,-rpath,$ORIGIN", "-o", KUIPER_TEST])
    return KUIPER_LIB


def build_kuiper_asan():
    """The C++ host API and its tests as one binary with AddressSanitizer on the host code (the device code
    is compiled as usual): lib/test_kuiper_asan.  Run it with ASAN_OPTIONS=protect_shadow_gap=0 (the HIP
    runtime maps memory where the sanitizer keeps a gap); at process exit the sanitizer's own allocator may
    trip over the already unloaded HIP runtime, after the tests have reported."""
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(LIB_DIR, "obj_asan")
    os.makedirs(obj_dir, exist_ok=True)
    inc = ["-I", INCLUDE, "-I", os.path.join(KUIPER, "include"), "-I", os.path.join(KUIPER, "source", "op"),
           "-I", TESTS_CPP]
    asan = ["-O1", "-g", "-std=c++17", "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fno-omit-frame-pointer"]
    srcs = sorted(glob.glob(os.path.join(KUIPER, "source", "**", "*.cpp"), recursive=True) +
                  glob.glob(os.path.join(KUIPER, "source", "**", "*.hip"), recursive=True) +
                  glob.glob(os.path.join(TESTS_CPP, "*.cpp")) + glob.glob(os.path.join(TESTS_CPP, "*.hip")))
    oracle_obj = os.path.join(obj_dir, "kx_oracle.o")
    _run(["gcc", "-O1", "-g", "-fPIC", "-std=c11", "-fsanitize=address", "-c",
          os.path.join(ROOT, "oracle", "kx_oracle.c"), "-o", oracle_obj])
    objs = [oracle_obj]
    for i, src in enumerate(srcs):
        obj = os.path.join(obj_dir, f"{i}_{os.path.basename(src)}.o")
        _run([HIPCC] + DEVICE_FLAGS + asan + inc + ["-c", src, "-o", obj])
        objs.append(obj)
    out = os.path.join(LIB_DIR, "test_kuiper_asan")
    _run([HIPCC, "--offload-arch=gfx950", "-fsanitize=address"] + objs +
         ["-L", LIB_DIR, "-lkx_hip", "-Wl,-rpath,$ORIGIN", "-o", out])
    return out


def build_all():
    build_kx()
    build_kuiper()
    build_probe()


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser()
    ap.add_argument("--ablate", type=int, default=0,
                    help="build lib/libkx_hip_ablateN.so (profiling only) and nothing else, so that several of these "
                         "builds can run side by side")
    ap.add_argument("--asan", action="store_true", help="also build lib/test_kuiper_asan (host code under AddressSanitizer)")
    args = ap.parse_args()
    if args.ablate:
        print("built:", build_kx(args.ablate))
        raise SystemExit(0)
    build_all()
    print("built:", KX_LIB, KUIPER_LIB if os.path.exists(KUIPER_LIB) else "", PROBE_LIB)
    if args.asan:
        print("built:", build_kuiper_asan())

"""Builds libsnn_hip.so (the HIP kernels + C ABI) in-tree with hipcc for gfx950.

    python -m portdnn_amd.build [-v] [--define NAME[=VALUE]]... [--output PATH]

--define adds a preprocessor definition (-DSNN_HIP_TUNING turns on the
developer switches read from the environment); --output writes the library
somewhere else than portdnn_amd/libsnn_hip.so, with its objects in a
directory of their own, and skips the C++ test programs.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libsnn_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=" + ARCH,
    "-fvisibility=hidden", "-Wall", "-Wextra", "-Wno-unused-parameter",
    # keep hipcc from fusing float pairs into packed-FP32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _compile(src, obj_dir=OBJ_DIR, defines=()):
    obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
    cmd = ([HIPCC] + FLAGS + ["-D" + d for d in defines] +
           ["-c", src, "-o", obj])
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, proc.stdout))
    return obj, out


def build_library(verbose=False, jobs=8, defines=(), output=None):
    """Compiles every csrc/*.hip and links libsnn_hip.so. Always rebuilds."""
    lib_path = LIB_PATH if output is None else os.path.abspath(output)
    obj_dir = OBJ_DIR if output is None else lib_path + ".objs"
    os.makedirs(obj_dir, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources under " + CSRC)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(
            lambda src: _compile(src, obj_dir, defines), sources))
    for obj, out in results:
        if verbose and out:
            print(out)
    objs = [obj for obj, _ in results]
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o",
           lib_path] + objs
    subprocess.check_call(cmd)
    return lib_path


CPP_TEST_DIR = os.path.join(ROOT, "tests", "cpp")


def build_cpp_tests():
    """Compiles the C++ programs under tests/cpp/ (users of the drop-in
    sycldnn:: headers) against libsnn_hip.so into tests/cpp/bin/."""
    sources = sorted(glob.glob(os.path.join(CPP_TEST_DIR, "*.cpp")))
    out_dir = os.path.join(CPP_TEST_DIR, "bin")
    built = []
    if not sources:
        return built
    os.makedirs(out_dir, exist_ok=True)
    for src in sources:
        exe = os.path.join(out_dir,
                           os.path.splitext(os.path.basename(src))[0])
        oracle_dir = os.path.join(ROOT, "oracle")
        # Host programs: the drop-in headers only need the HIP runtime API.
        cmd = ["g++", "-O2", "-std=c++17", "-Wall", "-Wextra",
               "-Wno-unused-parameter", "-I" + os.path.join(ROOT, "include"),
               "-I/opt/rocm/include", src, "-o", exe, "-L" + HERE,
               "-lsnn_hip", "-L" + oracle_dir, "-loracle",
               "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath," + HERE,
               "-Wl,-rpath," + oracle_dir, "-Wl,-rpath,/opt/rocm/lib"]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE,
                              stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, proc.stdout))
        built.append(exe)
    return built


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser()
    ap.add_argument("-v", action="store_true")
    ap.add_argument("--define", action="append", default=[])
    ap.add_argument("--output")
    a = ap.parse_args()
    print(build_library(verbose=a.v, defines=a.define, output=a.output))
    if a.output is None:
        print(build_cpp_tests())

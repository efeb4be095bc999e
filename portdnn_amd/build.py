"""Builds libsnn_hip.so (the HIP kernels + C ABI) in-tree with hipcc for gfx950.

    python -m portdnn_amd.build
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


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, proc.stdout))
    return obj, out


def build_library(verbose=False, jobs=8):
    """Compiles every csrc/*.hip and links libsnn_hip.so. Always rebuilds."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources under " + CSRC)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(_compile, sources))
    for obj, out in results:
        if verbose and out:
            print(out)
    objs = [obj for obj, _ in results]
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=" + ARCH, "-o",
           LIB_PATH] + objs
    subprocess.check_call(cmd)
    return LIB_PATH


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
    print(build_library(verbose="-v" in sys.argv))
    print(build_cpp_tests())

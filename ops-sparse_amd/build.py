"""Builds ops-sparse_amd/lib/libops_sparse.so for gfx950 with hipcc.

hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed:

    python ops-sparse_amd/build.py
    python ops-sparse_amd/build.py --asan     # host code under ASan / UBSan, then the CPU tests under it
    python ops-sparse_amd/build.py --coverage # a copy whose host code counts executed lines (see below)
    python ops-sparse_amd/build.py --kernel-coverage <dirs>   # kernels that traced test runs never launched

Every translation unit is compiled to an object under ops-sparse_amd/build/
(in parallel) and linked into one shared library.  The library carries both
the aclsparse* API (include/cann_ops_sparse.h) and the raw launch layer
(include/ops_sparse_hip.h).
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libops_sparse.so")

SOURCES = [
    "handle.cpp",
    "descr.cpp",
    "spmv_host.cpp",
    "spmv_op_host.cpp",
    "spmm_host.cpp",
    "convert_host.cpp",
    "spmv_kernels.hip",
    "spmv_blocked.hip",
    "spmv_blocked_live.hip",
    "spmv_scatter.hip",
    "spmm_kernels.hip",
    "convert_kernels.hip",
    "measure_kernels.hip",
]

# Packed fp32 VALU forms (v_pk_*_f32) are switched off for all device code.
COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"),
    "-I" + CSRC,
]


def hipcc():
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(path):
        raise RuntimeError("hipcc not found; ROCm is required to build libops_sparse.so")
    return path


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + COMMON_FLAGS
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # The host pass does not know the packed-fp32 feature name and says so; drop that line.
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build_library(verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        results = list(pool.map(_compile, SOURCES))
    for obj, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    objs = [obj for obj, _ in results]
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB_PATH] + objs
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    if verbose:
        print("built", LIB_PATH)
    return LIB_PATH


# ---- host code under AddressSanitizer / UndefinedBehaviorSanitizer -------------------------------------------------
# `python ops-sparse_amd/build.py --asan` builds a second copy of the library, of the CPU checker and of the C++
# frame's self-test with the HOST code instrumented (device code is compiled as always: no sanitizer runs on the
# GPU), and runs the tests that need no GPU under it: the status / argument tests of the C ABI, the checker's own
# tests, the frame's self-test.  Python itself is not instrumented, so the sanitizer runtime is preloaded.
ASAN_LIB_DIR = os.path.join(LIB_DIR, "asan")
ASAN_HOST = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined", "-Xarch_host",
             "-fno-omit-frame-pointer", "-g"]


def _clang_dir():
    out = subprocess.run([hipcc(), "-print-resource-dir"], capture_output=True, text=True).stdout.strip()
    if not out:
        out = subprocess.run([hipcc(), "--print-resource-dir"], capture_output=True, text=True).stdout.strip()
    return out


def asan_runtime():
    path = os.path.join(_clang_dir(), "lib", "linux", "libclang_rt.asan-x86_64.so")
    if not os.path.exists(path):
        raise RuntimeError("the sanitizer runtime %s is missing" % path)
    return path


def build_asan(verbose=True):
    obj_dir = OBJ_DIR + "_asan"
    os.makedirs(obj_dir, exist_ok=True)
    os.makedirs(ASAN_LIB_DIR, exist_ok=True)
    flags = [f if f != "-O3" else "-O1" for f in COMMON_FLAGS] + ASAN_HOST

    def compile_one(src):
        obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
        proc = subprocess.run([hipcc(), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + flags,
                              capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, proc.stderr))
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    lib = os.path.join(ASAN_LIB_DIR, "libops_sparse.so")
    link = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-sanitize", "-fsanitize=address",
            "-fsanitize=undefined", "-shared-libsan", "-o", lib] + objs
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    clang = os.path.join(_clang_dir().rstrip("/").rsplit("/lib/clang", 1)[0], "bin", "clang")  # (the hipcc's own)
    oracle_lib = os.path.join(ASAN_LIB_DIR, "liboracle.so")
    proc = subprocess.run([clang, "-O1", "-g", "-std=c99", "-fPIC", "-shared", "-ffp-contract=off", "-fopenmp",
                           "-fno-gpu-sanitize", "-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=undefined",
                           "-shared-libsan", "-fno-omit-frame-pointer", "-o", oracle_lib,
                           os.path.join(ROOT, "oracle", "oracle.c"), "-lm"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("the checker failed to build under the sanitizers:\n" + proc.stderr)
    selftest = os.path.join(ASAN_LIB_DIR, "frame_selftest")
    proc = subprocess.run([hipcc(), "-std=c++17", "-O1", "-g", "-fno-gpu-sanitize", "-fsanitize=address",
                           "-fsanitize=undefined", "-fno-sanitize-recover=undefined", "-shared-libsan",
                           "-I" + os.path.join(ROOT, "include"),
                           "-I" + os.path.join(ROOT, "tests", "cpp"),
                           os.path.join(ROOT, "tests", "cpp", "frame_selftest.cpp"), "-o", selftest,
                           "-L" + ASAN_LIB_DIR, "-lops_sparse", "-loracle", "-Wl,-rpath," + ASAN_LIB_DIR,
                           "-Wl,-rpath," + os.path.dirname(asan_runtime())], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("the frame's self-test failed to build under the sanitizers:\n" + proc.stderr)
    if verbose:
        print("built", lib, oracle_lib, selftest)
    return lib, oracle_lib, selftest


def run_asan():
    """The CPU tests with the instrumented libraries in place of the ordinary ones; returns the exit status."""
    lib, oracle_lib, selftest = build_asan()
    env = dict(os.environ)
    env["OPS_SPARSE_LIBRARY"] = lib
    env["OPS_SPARSE_ORACLE_LIBRARY"] = oracle_lib
    env["LD_PRELOAD"] = asan_runtime() + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    # (CPython and numpy keep their arenas until exit: no leak report; another preloaded library may come first)
    env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:abort_on_error=1"
    env["UBSAN_OPTIONS"] = "print_stacktrace=0:halt_on_error=0"
    names = ("test_abi_status.py", "test_launch_layer_status.py", "test_oracle.py", "test_oracle_convert.py")
    tests = [os.path.join(ROOT, "tests", t) for t in names]
    rc = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu"] + tests, env=env, cwd=ROOT).returncode
    if rc == 0:
        rc = subprocess.run([selftest, os.path.join(ROOT, "tests", "golden")], env=env).returncode
    return rc


# ---- which dispatch arms the tests reach ---------------------------------------------------------------------------
# `python ops-sparse_amd/build.py --coverage` builds lib/cov/libops_sparse.so with the HOST code counting executed
# lines (gcov format; device code as always).  Run any tests against it,
#     OPS_SPARSE_LIBRARY=ops-sparse_amd/lib/cov/libops_sparse.so GCOV_PREFIX=<dir> python -m pytest tests -m gpu
# (the counts are written at process exit below <dir>, or beside the objects without GCOV_PREFIX), then
# `python ops-sparse_amd/build.py --coverage-report <dir> [<dir> ...]` lists, per source file, the host lines that
# no run under any of the directories executed.
COV_LIB_DIR = os.path.join(LIB_DIR, "cov")
COV_OBJ_DIR = OBJ_DIR + "_cov"


def build_coverage(verbose=True):
    os.makedirs(COV_OBJ_DIR, exist_ok=True)
    os.makedirs(COV_LIB_DIR, exist_ok=True)
    flags = COMMON_FLAGS + ["-Xarch_host", "--coverage", "-Xarch_host", "-O0"]

    def compile_one(src):
        obj = os.path.join(COV_OBJ_DIR, os.path.splitext(src)[0] + ".o")
        proc = subprocess.run([hipcc(), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + flags,
                              capture_output=True, text=True, cwd=ROOT)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, proc.stderr))
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    lib = os.path.join(COV_LIB_DIR, "libops_sparse.so")
    runtime = os.path.join(_clang_dir(), "lib", "linux", "libclang_rt.profile-x86_64.a")
    proc = subprocess.run([hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-o", lib] + objs + [runtime],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    if verbose:
        print("built", lib)
    return lib


def coverage_report(count_dirs):
    """Sums the line counts of every run found below `count_dirs`; prints the host lines never executed."""
    import collections
    import glob
    import tempfile
    executed = collections.defaultdict(set)
    known = collections.defaultdict(dict)
    runs = []
    for d in count_dirs:
        for path in glob.glob(os.path.join(d, "**", "*.gcda"), recursive=True):
            runs.append(path)
    if not runs:
        print("no counts found below", count_dirs)
        return 1
    for gcda in runs:
        stem = os.path.splitext(os.path.basename(gcda))[0]
        gcno = os.path.join(COV_OBJ_DIR, stem + ".gcno")
        with tempfile.TemporaryDirectory() as tmp:
            shutil.copy(gcda, tmp)
            shutil.copy(gcno, tmp)
            os.symlink(HERE, os.path.join(tmp, os.path.basename(HERE)))    # the notes name sources relative to ROOT
            subprocess.run(["gcov", "-o", tmp, stem + ".o"], cwd=tmp, capture_output=True, text=True)
            for out in glob.glob(os.path.join(tmp, "*.gcov")):
                name = os.path.basename(out)[:-5]
                if not os.path.exists(os.path.join(CSRC, name)):
                    continue            # system and ROCm headers
                for line in open(out, errors="replace"):
                    parts = line.split(":", 2)
                    if len(parts) < 3:
                        continue
                    count, number = parts[0].strip(), int(parts[1])
                    if number == 0 or count == "-":
                        continue
                    known[name][number] = parts[2].rstrip("\n")
                    if count not in ("#####", "====="):
                        executed[name].add(number)
    total = missed = 0
    for name in sorted(known):
        lines = sorted(n for n in known[name] if n not in executed[name])
        total += len(known[name])
        missed += len(lines)
        print("%s: %d of %d host lines never executed" % (name, len(lines), len(known[name])))
        for n in lines:
            print("    %5d:%s" % (n, known[name][n]))
    print("total: %d of %d host lines never executed" % (missed, total))
    return 0


def kernel_coverage(trace_dirs):
    """Which kernel instantiations of the built library no traced run launched.  `trace_dirs` hold the
    `*kernel_stats.csv` files of `rocprofv3 --kernel-trace --stats -M --output-format csv -d <dir> -- python3 -m pytest
    tests/<file> -m gpu` runs (-M: mangled names, which is what the library's symbol table has)."""
    import csv
    import glob
    import re
    out = subprocess.run(["nm", LIB_PATH], capture_output=True, text=True, check=True).stdout
    compiled = set()
    for line in out.splitlines():
        m = re.search(r"\s(_Z\S*?)(\d+)__device_stub__(\S+)$", line)
        if m:  # the host stub of a kernel: its name with "__device_stub__" in front of the last component
            compiled.add(m.group(1) + str(int(m.group(2)) - len("__device_stub__")) + m.group(3))
    launched = set()
    for d in trace_dirs:
        for path in glob.glob(os.path.join(d, "**", "*kernel_stats.csv"), recursive=True):
            with open(path, newline="") as f:
                for row in csv.DictReader(f):
                    launched.add(row["Name"].replace(".kd", ""))
    missing = sorted(compiled - launched)
    print("%d kernel instantiations in %s, %d of them never launched by the traced runs" %
          (len(compiled), os.path.relpath(LIB_PATH, ROOT), len(missing)))
    if missing:
        shown = subprocess.run(["c++filt"], input="\n".join(missing), capture_output=True, text=True).stdout
        print(shown.rstrip())
    return 1 if missing else 0


if __name__ == "__main__":
    if "--kernel-coverage" in sys.argv[1:]:
        sys.exit(kernel_coverage(sys.argv[sys.argv.index("--kernel-coverage") + 1:]))
    if "--asan" in sys.argv[1:]:
        sys.exit(run_asan())
    if "--coverage" in sys.argv[1:]:
        build_coverage()
        sys.exit(0)
    if "--coverage-report" in sys.argv[1:]:
        sys.exit(coverage_report(sys.argv[sys.argv.index("--coverage-report") + 1:]))
    build_library()

"""The C side of the boundary: the public headers compile as plain C, and a C++ caller written against
cann_ops_sparse.h only (tests/cpp/run_case_tables.cpp, with the small RAII / CSV frame of tests/cpp/frame.h)
runs the reference's case tables on the GPU.  The runner is built by `make -C tests/cpp`
(__graft_entry__.build() does it)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
RUNNER = os.path.join(ROOT, "tests", "cpp", "bin", "run_case_tables")


def test_headers_compile_as_c99():
    proc = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only",
                           "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "cpp", "abi_c_compile.c")],
                          capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr


def test_frame_rules_and_typed_loader_on_the_cpu():
    """tests/cpp/frame_selftest: the C++ verification rules against the C checker and hand-computed values, and
    GetCasesFromCsv<T> on the 70-row SpMVOp table.  Makes no GPU call."""
    selftest = os.path.join(ROOT, "tests", "cpp", "bin", "frame_selftest")
    if not os.path.exists(selftest):
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "cpp"), "bin/frame_selftest"], check=True,
                       capture_output=True)
    proc = subprocess.run([selftest, os.path.join(ROOT, "tests", "golden")], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 0 and "0 failed" in proc.stdout, proc.stdout + proc.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("table", ["spmv_op", "coo2csr", "csr2coo", "csr2csc", "csrsort", "cscsort", "coosort"])
def test_case_tables_from_cpp(gpu_ctx, table):
    assert os.path.exists(RUNNER), "tests/cpp/bin/run_case_tables is not built: run `make -C tests/cpp`"
    proc = subprocess.run([RUNNER, os.path.join(ROOT, "tests", "golden"), table], capture_output=True, text=True,
                          timeout=110)
    tail = "\n".join(proc.stdout.splitlines()[-12:])
    assert proc.returncode == 0, tail + "\n" + proc.stderr[-2000:]
    assert ", 0 failed" in proc.stdout

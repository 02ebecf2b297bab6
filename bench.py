#!/usr/bin/env python3
"""Benchmark of the CSR SpMV / SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|c2|c3|c4|c5|convert|cache]

A step is one aclsparseSpMV (or aclsparseSpMM) call over one synthetic matrix
whose arrays are already resident in HBM.  The headline workload is c2, the
5-point 2-D Laplacian on a 2048 x 2048 grid (m = n = 4 194 304, nnz = 20 963 328,
alpha = 1, beta = 0.5), the configuration the headline metric is quoted on; its
238 MB fit the 256 MB Infinity Cache, so its launches go round three independent
copies of the operands (the figure on one copy is kept as roofline.warm).  With
the default --workload all the other measured configurations follow in the same
run and land in the `workloads` object: c3 (power-law SpMV; default plan and the
ALG2 layout), c4 (fp32 SpMM) and c5 (fp16 SpMM), each with its own roofline and
CPU baseline.  Preprocess runs once before the timed region (its time is
reported separately).  Timing: rounds of K launches between two HIP events on
the handle's stream, repeated until 50 ms of GPU time; the median round counts.

Prints ONE JSON line: GFLOP/s = 2 * nnz * ncols / t as `value`, the roofline
object (algorithmic bytes / kernel time against 8 TB/s HBM) and the CPU baseline
(the reference's CPU golden loop restated in oracle/, timed on this host).
--workload convert times the CSR producers instead (its own JSON line); --workload cache is the Infinity-Cache
probe: the copy / read yard-sticks by buffer size, and the c4 product with the rows of B it gathers confined to a
window of B.
"""
import argparse
import ctypes
import importlib
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak


def load_package():
    if "ops_sparse_amd" in sys.modules:
        return sys.modules["ops_sparse_amd"]
    pkg_dir = os.path.join(ROOT, "ops-sparse_amd")
    spec = importlib.util.spec_from_file_location(
        "ops_sparse_amd", os.path.join(pkg_dir, "__init__.py"), submodule_search_locations=[pkg_dir])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["ops_sparse_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def _time_launches(torch, stream, launch, reps):
    for _ in range(2):
        launch()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        launch()
    e1.record(stream)
    stream.synchronize()
    return e0.elapsed_time(e1) / reps * 1e-3


def measure_yardsticks(osa, torch, dev, stream, nbytes=1 << 30, reps=10):
    """Practical HBM peaks of this GPU: a >= 1 GiB device-to-device copy, (read + write) / t,
    and a read-only pass over the same buffer."""
    src = torch.empty(nbytes, dtype=torch.uint8, device=dev).zero_()
    dst = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    L = osa.lib()
    sp = ctypes.c_void_p(stream.cuda_stream)
    torch.cuda.synchronize()
    t_copy = _time_launches(torch, stream, lambda: L.opsparse_copy_launch(src.data_ptr(), dst.data_ptr(), nbytes, sp),
                            reps)
    t_read = _time_launches(torch, stream, lambda: L.opsparse_read_launch(src.data_ptr(), nbytes, None, sp), reps)
    return 2.0 * nbytes / t_copy / 1e9, nbytes / t_read / 1e9


def measure_gather(osa, torch, wl, dev, stream, count=1 << 26):
    """Random 4-byte gathers per second from vectors of 4 MiB, 32 MiB and 256 MiB."""
    L = osa.lib()
    sp = ctypes.c_void_p(stream.cuda_stream)
    out = {}
    for mib in (4, 32, 256):
        nx = mib << 18
        x = torch.zeros(nx, dtype=torch.float32, device=dev)
        idx = (wl._lsr(wl.hash64(77, torch.arange(count, dtype=torch.int64, device=dev)), 11) % nx).to(torch.int32)
        torch.cuda.synchronize()
        t = _time_launches(torch, stream, lambda: L.opsparse_gather_launch(idx.data_ptr(), x.data_ptr(), count, None,
                                                                           sp), 5)
        out["x_%dMiB" % mib] = round(count / t / 1e9, 2)
    return out


def load_traffic(name):
    """Measured HBM traffic per launch for a workload, from the committed rocprof summary."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        table = json.load(f)
    entry = table.get("workloads", {}).get(name)
    if entry is None:
        return None
    return int(entry["fetch_kib"] * 1024 * table["fetch_scale"] + entry["write_kib"] * 1024 * table["write_scale"])


def cpu_baseline_spmv(cfg, y_gpu, base=None, budget_s=15.0, transpose=False):
    """The reference's SpmvCpu loop (oracle.spmv_f32; op(A) = A^T: its SpmvTransCpu, oracle.spmv_trans_f32,
    reference test/spmv/arch22/spmv_test.cpp:177-197), one thread, on the same matrix; the GPU result of one
    launch (y_gpu) is checked against the fp64-accumulated oracle on the way.  `base` is the result of an earlier
    call on the same matrix: the CPU timing is taken from it and only the check is repeated."""
    import oracle
    A = cfg["A"]
    rowptr, colind = A["rowptr"].cpu().numpy(), A["colind"].cpu().numpy()
    val = A["values"].cpu().float().numpy()
    x, y0 = cfg["x"].cpu().float().numpy(), cfg["y0"].cpu().float().numpy()
    rows, cols, nnz = A["rows"], A["cols"], int(colind.size)
    if transpose:
        gold = oracle.spmv_trans_f64(rows, cols, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"])
        cpu = lambda: oracle.spmv_trans_f32(rows, cols, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"])
        name = "SpmvTransCpu"
    else:
        gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"])
        cpu = lambda: oracle.spmv_f32(rows, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"])
        name = "SpmvCpu"
    err = oracle.max_rel_err(y_gpu.cpu().numpy(), gold)
    if err > 1e-5:
        sys.exit("bench.py: the GPU result differs from the fp64 oracle (max relative error %.3g > 1e-5)" % err)
    if base is not None:
        return dict(base, gpu_vs_fp64_oracle_max_rel_err=err)
    cpu()  # warm
    reps, t0 = 0, time.perf_counter()
    while reps < 10 and time.perf_counter() - t0 < budget_s:
        cpu()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    res = {"value": 2.0 * nnz / dt / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
           "sample": "full matrix, %d repeats of the reference's %s loop restated in oracle/oracle.c "
                     "(fp32 accumulate), %.1f ms each" % (reps, name, dt * 1e3),
           "gpu_vs_fp64_oracle_max_rel_err": err}
    if not transpose:
        # the same loop with its rows shared out among all host threads (second baseline, reported beside the first)
        threads = oracle.host_threads()
        oracle.spmv_f32_threads(rows, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"], threads)
        t0 = time.perf_counter()
        for _ in range(5):
            oracle.spmv_f32_threads(rows, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"], threads)
        dt_all = (time.perf_counter() - t0) / 5
        res["all_cores"] = {"value": 2.0 * nnz / dt_all / 1e9, "unit": "GFLOP/s", "cores": threads,
                            "sample": "the same loop, rows shared out among %d OpenMP threads, %.1f ms each"
                                      % (threads, dt_all * 1e3)}
    return res


def cpu_baseline_spmm(cfg, c_gpu, base=None, rows_sample=262144):
    """The reference's spmm_csr_cpu loop (order i, j, p) on the first rows_sample rows; the same rows of the GPU
    result of one launch (c_gpu) are checked against the fp64-accumulated oracle on the way."""
    import oracle
    A = cfg["A"]
    n = cfg["n"]
    rs = min(rows_sample, A["rows"])
    rowptr = A["rowptr"][: rs + 1].cpu().numpy()
    nnz = int(rowptr[-1])
    colind = A["colind"][:nnz].cpu().numpy()
    val = A["values"][:nnz].cpu().float().numpy()
    B = cfg["B"].cpu().float().numpy()
    import numpy as np
    C = np.zeros(rs * n, np.float32)
    t0 = time.perf_counter()
    oracle.spmm_f32(rs, n, rowptr, colind, val, B.ravel(), n, C, n, cfg["alpha"], cfg["beta"])
    dt = time.perf_counter() - t0
    gold = oracle.spmm_f64_rowmajor(rs, n, rowptr, colind, val, B, n, np.zeros((rs, n), np.float32), n, cfg["alpha"],
                                    cfg["beta"])
    err = oracle.max_rel_err(c_gpu[:rs].cpu().numpy(), np.asarray(gold))
    tol = 1e-5 if A["values"].element_size() == 4 else 1e-3
    if err > tol:
        sys.exit("bench.py: the GPU result differs from the fp64 oracle (max relative error %.3g > %g)" % (err, tol))
    threads = oracle.host_threads()
    t0 = time.perf_counter()
    oracle.spmm_f32_threads(rs, n, rowptr, colind, val, B.ravel(), n, C, n, cfg["alpha"], cfg["beta"], threads)
    dt_all = time.perf_counter() - t0
    return {"value": 2.0 * nnz * n / dt / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
            "sample": "first %d of %d rows (%d nnz) against the full B, one run of the reference's "
                      "SpmmCpuFp32 loop restated in oracle/oracle.c, %.1f s" % (rs, A["rows"], nnz, dt),
            "all_cores": {"value": 2.0 * nnz * n / dt_all / 1e9, "unit": "GFLOP/s", "cores": threads,
                          "sample": "the same rows and loop shared out among %d OpenMP threads, %.2f s"
                                    % (threads, dt_all)},
            "gpu_vs_fp64_oracle_max_rel_err": err}


def vendor_yardstick(torch, cfg, is_spmm, flops, bytes_alg, steps, stream, ours):
    """The same product through rocSPARSE's generic API (rocsparse_spmv / rocsparse_spmm: buffer size and
    preprocess once, then `steps` compute calls between two events on `stream`), for each of its CSR
    algorithms.  A yard-stick beside the figures, not an oracle; `ours` is this library's result for beta = 0,
    and one more call with beta = 0 is compared with it so that an algorithm that did nothing is not quoted."""
    import ctypes
    try:
        rs = ctypes.CDLL("librocsparse.so.1")
    except OSError as exc:
        return {"error": str(exc)}
    vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    I32, F16, F32, NONE, ROW = 2, 150, 151, 111, 0  # rocsparse_indextype / datatype / operation / order values
    rs.rocsparse_create_csr_descr.argtypes = [ctypes.POINTER(vp), i64, i64, i64, vp, vp, vp, ci, ci, ci, ci]
    rs.rocsparse_create_dnvec_descr.argtypes = [ctypes.POINTER(vp), i64, vp, ci]
    rs.rocsparse_create_dnmat_descr.argtypes = [ctypes.POINTER(vp), i64, i64, i64, vp, ci, ci]
    rs.rocsparse_set_stream.argtypes = [vp, vp]
    rs.rocsparse_spmv.argtypes = [vp, ci, vp, vp, vp, vp, vp, ci, ci, ci, ctypes.POINTER(ctypes.c_size_t), vp]
    rs.rocsparse_spmm.argtypes = [vp, ci, ci, vp, vp, vp, vp, vp, ci, ci, ci, ctypes.POINTER(ctypes.c_size_t), vp]
    A = cfg["A"]
    rows, cols, nnz = A["rows"], A["cols"], int(A["colind"].numel())
    vt = F32 if A["values"].element_size() == 4 else F16
    handle, mat, dx, dy = vp(), vp(), vp(), vp()
    if rs.rocsparse_create_handle(ctypes.byref(handle)):
        return {"error": "rocsparse_create_handle failed"}
    rs.rocsparse_set_stream(handle, vp(stream.cuda_stream))
    rs.rocsparse_create_csr_descr(ctypes.byref(mat), rows, cols, nnz, A["rowptr"].data_ptr(), A["colind"].data_ptr(),
                                  A["values"].data_ptr(), I32, I32, 0, vt)
    if is_spmm:
        n = cfg["n"]
        dense = cfg["B"].contiguous()
        out = torch.zeros(rows, n, dtype=torch.float32, device=dense.device)
        rs.rocsparse_create_dnmat_descr(ctypes.byref(dx), cols, n, n, dense.data_ptr(), vt, ROW)
        rs.rocsparse_create_dnmat_descr(ctypes.byref(dy), rows, n, n, out.data_ptr(), F32, ROW)
        algs = {"default": 0, "csr": 1, "csr_row_split": 4, "csr_nnz_split": 5, "csr_merge_path": 9}
    else:
        dense = cfg["x"]
        out = cfg["y0"].clone()
        rs.rocsparse_create_dnvec_descr(ctypes.byref(dx), cols, dense.data_ptr(), vt)
        rs.rocsparse_create_dnvec_descr(ctypes.byref(dy), rows, out.data_ptr(), F32)
        algs = {"default": 0, "csr_adaptive": 2, "csr_rowsplit": 3, "csr_lrb": 7, "csr_nnzsplit": 8}
    alpha, beta, zero = ctypes.c_float(cfg["alpha"]), ctypes.c_float(cfg["beta"]), ctypes.c_float(0.0)
    scale = float(ours.abs().max().item()) or 1.0

    def call(alg, stage, size, buf, b=beta):
        if is_spmm:
            return rs.rocsparse_spmm(handle, NONE, NONE, ctypes.byref(alpha), mat, dx, ctypes.byref(b), dy, F32,
                                     alg, stage, ctypes.byref(size), buf)
        return rs.rocsparse_spmv(handle, NONE, ctypes.byref(alpha), mat, dx, ctypes.byref(b), dy, F32, alg, stage,
                                 ctypes.byref(size), buf)

    res = {"what": "rocsparse_%s, buffer size and preprocess once, %d compute calls per algorithm"
                   % ("spmm" if is_spmm else "spmv", steps)}
    for name, alg in algs.items():
        size = ctypes.c_size_t(0)
        st = call(alg, 1, size, None)
        buf = torch.empty(max(int(size.value), 256), dtype=torch.uint8, device=dense.device)
        st = st or call(alg, 2, size, vp(buf.data_ptr()))
        st = st or call(alg, 3, size, vp(buf.data_ptr()))
        stream.synchronize()
        if st:
            res[name] = {"status": st}
            continue
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps):
            call(alg, 3, size, vp(buf.data_ptr()))
        e1.record(stream)
        stream.synchronize()
        ms = e0.elapsed_time(e1) / steps
        out.zero_()  # not NaN: some of the vendor's kernels scale y by beta = 0 before they add to it
        call(alg, 3, size, vp(buf.data_ptr()), zero)
        stream.synchronize()
        diff = float(((out - ours).abs().max() / scale).item())
        if not diff <= 1e-3:
            res[name] = {"error": "result differs from this library's (max |d| / max |ours| = %g): not quoted" % diff,
                         "ms_per_step": round(ms, 6)}
            continue
        res[name] = {"ms_per_step": round(ms, 6), "value": round(flops / (ms * 1e-3) / 1e9, 2), "unit": "GFLOP/s",
                     "frac_of_8TBs": round(bytes_alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                     "buffer_bytes": int(size.value), "max_diff_vs_ours": diff}
    return res


def time_rounds(torch, stream, launch, steps, restore=None, min_gpu_ms=50.0, min_rounds=5, max_rounds=2000):
    """Rounds of `steps` back-to-back launches, each between two HIP events recorded on `stream` (the stream the
    kernels run on), repeated until `min_gpu_ms` of GPU time has been timed.  `launch(i)` gets the running launch
    number; `restore()` runs before every round, outside the timed region (y back to y0 when beta != 0).
    Returns per-step milliseconds (median round, fastest round, mean, number of rounds) and what a reader needs to
    judge the spread: the slowest round, how many rounds took more than 1.5 x the median, and, for those, the time
    the HOST spent inside the round's launch calls (a round that is slow because a launch call blocked the host shows
    it there: the GPU then idles between the two events)."""
    per_step, host_ms, total, i = [], [], 0.0, 0
    while (total < min_gpu_ms or len(per_step) < min_rounds) and len(per_step) < max_rounds:
        if restore is not None:
            restore()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        t0 = time.perf_counter()
        for _ in range(steps):
            launch(i)
            i += 1
        host_ms.append((time.perf_counter() - t0) * 1e3)
        e1.record(stream)
        stream.synchronize()
        ms = e0.elapsed_time(e1)
        per_step.append(ms / steps)
        total += ms
    if os.environ.get("BENCH_LOG_ROUNDS"):
        log("rounds (ms per step, in order): " + " ".join("%.4f" % v for v in per_step))
        log("host ms inside the launch calls, per round: " + " ".join("%.2f" % v for v in host_ms))
    s = sorted(per_step)
    median = s[len(s) // 2]
    slow = [k for k, v in enumerate(per_step) if v > 1.5 * median]
    spread = {"rounds": len(s), "slowest_round_ms_per_step": round(s[-1], 6),
              "rounds_over_1p5x_median": len(slow),
              "slow_rounds": [{"round": k, "ms_per_step": round(per_step[k], 6),
                               "host_ms_in_launch_calls": round(host_ms[k], 3),
                               "gpu_ms": round(per_step[k] * steps, 3)} for k in slow[:4]]}
    return median, s[0], sum(s) / len(s), len(s), spread


WORKLOADS = {
    # key: (generator config, layout asked for, op(A) = A^T, environment of the run)
    "c2": ("c2", "csr", False, {}),
    "c3": ("c3", "csr", False, {}),
    "c3_repeatable": ("c3", "csr", False, {"OPS_SPARSE_SPMV_REPEATABLE": "1"}),
    "c3_transposed": ("c3", "csr", True, {}),
    "c3_alg2": ("c3", "blocked_gather", False, {}),
    "c3_panels": ("c3", "column_panels", False, {"OPS_SPARSE_SPMV_NO_BLOCKED": "1"}),
    "c4": ("c4", "csr", False, {}),
    "c5": ("c5", "csr", False, {}),
}
BENCH_ENV = ("OPS_SPARSE_SPMV_NO_BLOCKED", "OPS_SPARSE_SPMV_REPEATABLE", "OPS_SPARSE_SPMV_NO_SCATTER",
             "OPS_SPARSE_SCATTER_MIN_PANELS", "OPS_SPARSE_SPMV_NO_DEFAULT_BLOCKED", "OPS_SPARSE_ORDERED_LIVE_MIN_COLS",
             "OPS_SPARSE_BLOCKED_NO_STREAM")
_cfg_cache = {}


def make_config(wl, torch, dev, which, scale):
    """The synthetic operands of one configuration, kept until another configuration is asked for (the two c3
    entries share one matrix)."""
    key = (which, scale)
    if key in _cfg_cache:
        return _cfg_cache[key]
    _cfg_cache.clear()
    torch.cuda.empty_cache()
    s = scale
    t_gen = time.perf_counter()
    if which == "c2":
        cfg = wl.config_c2(dev, grid=max(8, int(2048 * s ** 0.5)))
    elif which == "c3":
        cfg = wl.config_c3(dev, m=max(1024, int(8388608 * s)), lmax=200000 if s >= 0.05 else 2000)
    elif which == "c4":
        cfg = wl.config_c4(dev, m=max(1024, int(1048576 * s)))
    else:
        cfg = wl.config_c5(dev, m=max(1024, int(2097152 * s)))
    torch.cuda.synchronize()
    log("workload %s: rows=%d nnz=%d (generated in %.1f s)"
        % (cfg["name"], cfg["A"]["rows"], int(cfg["A"]["colind"].numel()), time.perf_counter() - t_gen))
    _cfg_cache[key] = cfg
    return cfg


def run_workload(args, osa, wl, torch, dev, stream, handle, key, cpu_cache):
    """One workload: Preprocess once, then rounds of `--steps` calls; returns the fields of its JSON object."""
    which, layout, transpose, env = WORKLOADS[key]
    for name in BENCH_ENV:
        os.environ.pop(name, None)
    os.environ.update(env)
    cfg = make_config(wl, torch, dev, which, args.scale)
    A = cfg["A"]
    rows, cols, nnz = A["rows"], A["cols"], int(A["colind"].numel())
    is_spmm = "B" in cfg
    vb = A["values"].element_size()
    alpha, beta = cfg["alpha"], cfg["beta"]
    # Operand sets.  A timed loop over ONE set re-reads the same bytes every launch; when they fit the 256 MB
    # Infinity Cache (c2: 238 MB) part of them never comes from HBM.  The headline of such a workload is therefore
    # timed over `nsets` independent copies of (A, x, y) used in turn, 3 x 238 MB, and the figure on one set is
    # kept beside it as `warm`.
    footprint = sum(t.numel() * t.element_size() for t in (A["rowptr"], A["colind"], A["values"]))
    footprint += sum(cfg[k].numel() * cfg[k].element_size() for k in ("x", "y0", "B") if k in cfg)
    nsets = 1 if (footprint > 400e6 or args.warm_only) else 3
    sets = []
    t_pre = time.perf_counter()
    first_use_ms = preprocess_ms = None
    for s in range(nsets + 1):  # set 0 is built twice: the first build also loads the kernels onto the device
        if s <= 1:
            arrs = (A["rowptr"], A["colind"], A["values"])
        else:
            arrs = tuple(t.clone() for t in (A["rowptr"], A["colind"], A["values"]))
        csr = osa.Csr(rows, cols, *arrs)
        stream.synchronize()
        t_pre = time.perf_counter()
        if not is_spmm:
            # (op(A) = A^T: the configurations are square, x and y0 serve as they are)
            x = cfg["x"] if s <= 1 else cfg["x"].clone()
            y = cfg["y0"].clone()
            X, Y = osa.DnVec(x), osa.DnVec(y)
            op = osa.SpmvOp(handle, csr, X, Y, preprocess=not args.no_preprocess,
                            op=osa.ACL_SPARSE_OP_TRANSPOSE if transpose else osa.ACL_SPARSE_OP_NON_TRANSPOSE,
                            alg=osa.ACL_SPARSE_SPMV_CSR_ALG2 if layout != "csr" else osa.ACL_SPARSE_SPMV_ALG_DEFAULT)
            out_t = y
        else:
            n = cfg["n"]
            B = cfg["B"].contiguous() if s <= 1 else cfg["B"].clone()
            Cmat = torch.zeros(rows, n, dtype=torch.float32, device=dev)
            op = osa.SpmmOp(handle, csr, osa.DnMat(cols, n, n, B), osa.DnMat(rows, n, n, Cmat))
            out_t = Cmat
        stream.synchronize()
        dt = (time.perf_counter() - t_pre) * 1e3
        if s == 0:
            first_use_ms = dt       # includes loading the library's kernels onto the device
            continue
        if s == 1:
            preprocess_ms = dt      # GetBufferSize + buffer allocation + Preprocess: what a second matrix costs
        sets.append((op, out_t))
    if not is_spmm:
        # which plan Preprocess chose shows in the buffer it asked for
        L = osa.lib()
        got = sets[0][0].buffer.numel() if sets[0][0].buffer is not None else 0
        tflag = osa.OPSPARSE_BLOCKED_TRANSPOSE if transpose else 0
        frozen = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, tflag)
        ordered_live = L.opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz,
                                                                   tflag | osa.OPSPARSE_BLOCKED_LIVE_VALUES)
        atomics_live = 0 if transpose else L.opsparse_spmv_csr_live_workspace_bytes(rows, cols, nnz)
        if layout == "blocked_gather" and not (frozen and got == frozen):
            layout = "column_panels" if L.opsparse_spmv_csr_panels_workspace_bytes(rows, cols, nnz) else "csr"
        resident = None
        if layout == "blocked_gather":
            resident = L.opsparse_spmv_csr_blocked_resident_bytes(rows, cols, nnz, tflag)
        elif layout == "csr" and atomics_live and got == atomics_live:
            # the default algorithm found the gathers scattered: live values, row blocks summed with LDS atomics
            layout = "blocked_live_atomics"
            resident = L.opsparse_spmv_csr_live_resident_bytes(rows, cols, nnz)
        elif layout == "csr" and ordered_live and got == ordered_live:
            # ... or the same with every row summed in a fixed order (asked for, op(A) = A^T, int32)
            layout = "blocked_gather_live_values"
            resident = L.opsparse_spmv_csr_blocked_resident_bytes(rows, cols, nnz,
                                                                  tflag | osa.OPSPARSE_BLOCKED_LIVE_VALUES)
            scatter = L.opsparse_spmv_csr_scatter_resident_bytes(rows, cols, nnz, 0) if transpose else 0
            if scatter and "OPS_SPARSE_SPMV_REPEATABLE" not in os.environ and "OPS_SPARSE_SPMV_NO_SCATTER" not in os.environ:
                # op(A) = A^T where the last bit may vary: inside the same buffer Preprocess builds the layout that
                # sorts the products by output panel (no column of the benchmark matrices is full enough to refuse it)
                layout = "scatter_live"
                resident = scatter
        ncols = 1
        bytes_alg = wl.spmv_bytes_alg(rows, cols, nnz, vb, 4, 4, beta != 0)
        bytes_gather = wl.spmv_bytes_gather(rows, cols, nnz, vb, 4, 4, beta != 0)
        dtype = "f32"
    else:
        ncols = cfg["n"]
        eb = cfg["B"].element_size()
        bytes_alg = wl.spmm_bytes_alg(rows, cols, ncols, nnz, vb, eb, 4, beta != 0)
        bytes_gather = wl.spmm_bytes_gather(rows, cols, ncols, nnz, vb, eb, 4, beta != 0)
        dtype = "f32" if vb == 4 else "f16 in, f32 accumulate/out"

    # the buffer Preprocess was given and, for the blocked-gather layouts, the part of it the launches need
    buf = getattr(sets[0][0], "buffer", None)
    buffer_mib = round(buf.numel() / 2.0 ** 20, 1) if buf is not None else 0.0
    resident_mib = buffer_mib
    if not is_spmm and resident is not None:
        resident_mib = round(resident / 2.0 ** 20, 1)

    def restore():
        if beta != 0:  # y back to y0 before every round, outside the timed region
            for _, t in sets:
                t.copy_(cfg["y0"])

    restore()
    sets[0][0](alpha, beta)  # one launch from the initial y / C, kept for the check against the fp64 oracle
    stream.synchronize()
    first_result = sets[0][1].clone()
    for i in range(args.warmup):
        sets[i % len(sets)][0](alpha, beta)
    stream.synchronize()
    # Settling, untimed like the warm-up: the HIP runtime blocks the host for some 30 ms inside one launch call
    # around a process's 330th kernel launch (and for 1 ms around the 170th) while it grows one of its pools, and
    # the GPU's clocks take some 200 launches of this size to settle.  Both are one-off: left in the timed
    # region they cost most of its 50 ms budget and put the median on the unsettled rounds.
    for i in range(args.settle):
        sets[i % len(sets)][0](alpha, beta)
    stream.synchronize()
    ms, ms_min, ms_mean, nrounds, spread = time_rounds(torch, stream, lambda i: sets[i % len(sets)][0](alpha, beta),
                                                       args.steps, restore, args.min_gpu_ms)
    warm = None
    if len(sets) > 1:
        w_ms, w_min, _, _, _ = time_rounds(torch, stream, lambda i: sets[0][0](alpha, beta), args.steps, restore,
                                        args.min_gpu_ms)
        warm = {"ms_per_step": round(w_ms, 6), "ms_per_step_min": round(w_min, 6),
                "achieved": round(bytes_alg / (w_ms * 1e-3) / 1e9, 1),
                "frac": round(bytes_alg / (w_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                "what": "every launch on the same operand set (%.0f MB, inside the 256 MB Infinity Cache)"
                        % (footprint / 1e6)}
    flops = 2.0 * nnz * ncols
    gflops = flops / (ms * 1e-3) / 1e9
    gbps = bytes_alg / (ms * 1e-3) / 1e9
    log("%-9s %.2f us/step (median of %d rounds of %d; fastest %.2f, mean %.2f), %.1f GFLOP/s, %.1f GB/s algorithmic "
        "= %.1f%% of 8 TB/s%s"
        % (key, ms * 1e3, nrounds, args.steps, ms_min * 1e3, ms_mean * 1e3, gflops, gbps, 100 * gbps / HBM_PEAK_GBPS,
           "; same operands every launch %.2f us = %.1f%%" % (warm["ms_per_step"] * 1e3, 100 * warm["frac"])
           if warm else ""))
    traffic = load_traffic(cfg["name"] + ("+" + layout if layout != "csr" else "") +
                           ("+transposed" if transpose else "")) if args.scale == 1.0 else None
    out = {
        "value": round(gflops, 2), "unit": "GFLOP/s", "ms_per_step": round(ms, 6),
        "ms_per_step_min": round(ms_min, 6), "ms_per_step_mean": round(ms_mean, 6), "rounds": nrounds,
        "round_spread": spread,
        "dtype": dtype,
        "config": {"workload": cfg["name"], "rows": rows, "cols": cols, "nnz": nnz, "ncols_dense": ncols,
                   "alpha": alpha, "beta": beta, "index": "int32", "preprocess_ms": round(preprocess_ms, 3),
                   "first_use_ms": round(first_use_ms, 3), "preprocessed": not args.no_preprocess, "layout": layout,
                   "operand_sets": len(sets), "buffer_mib": buffer_mib, "buffer_resident_mib": resident_mib,
                   "op": "transpose" if transpose else "non_transpose",
                   "timing": "median over rounds of `steps` launches between HIP events on the handle's stream, "
                             "rounds repeated until %.0f ms of GPU time, after `warmup` + %d untimed launches%s" % (
                                 args.min_gpu_ms, args.settle,
                                 "; y restored to y0 before every round" if beta != 0 else "")},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     "traffic": traffic,
                     "traffic_gbps": round(traffic / (ms * 1e-3) / 1e9, 1) if traffic else None,
                     "bytes_alg": bytes_alg, "bytes_gather_model": bytes_gather,
                     # the dense operand counted once per use instead of once: what a row-wise kernel has to move
                     # when none of its gathers hits a cache (never the headline figure: it credits cache hits)
                     "gather_model_gbps": round(bytes_gather / (ms * 1e-3) / 1e9, 1)},
    }
    if warm:
        out["roofline"]["warm"] = warm
    if args.vendor and not transpose:  # (the vendor call below is made for op(A) = A)
        sets[0][0](alpha, 0.0)
        stream.synchronize()
        out["vendor_yardstick"] = vendor_yardstick(torch, cfg, is_spmm, flops, bytes_alg, max(5, args.steps // 4),
                                                   stream, sets[0][1].clone())
    if not args.no_cpu:
        ck = which + ("_t" if transpose else "")
        base = cpu_cache.get(ck)
        res = (cpu_baseline_spmm(cfg, first_result, base) if is_spmm else
               cpu_baseline_spmv(cfg, first_result, base, transpose=transpose))
        cpu_cache[ck] = res
        out["cpu_baseline"] = res
        out["gpu_vs_fp64_oracle_max_rel_err"] = res["gpu_vs_fp64_oracle_max_rel_err"]
    del sets
    return out


def run_c1(args, osa, torch, dev, stream, handle):
    """The reference's own CPU-runnable case: m = n = 4096, 16 entries a row from the reference's generator
    (SparseFillGenerator, seed 42: reference test/frame/fill.h:71-111), values and x ~ U(-1, 1), alpha = 1,
    beta = 0.  65 536 entries are 0.8 MB: a call is bound by launch latency, not bandwidth, so the entry gives
    microseconds per call (with and without Preprocess) beside the time of the reference's SpmvCpu loop, and no
    roofline.  The generator and the CPU loop are the oracle's: this entry is part of the CPU-baseline leg."""
    import numpy as np
    import oracle
    rows = cols = 4096
    rowptr, colind, val = oracle.fill_csr(42, rows, cols, rows * 16, -1.0, 1.0)
    x = oracle.fill_dense(43, cols, -1.0, 1.0)
    nnz = int(colind.size)
    d = [torch.from_numpy(a).to(dev) for a in (rowptr, colind, val, x)]
    csr = osa.Csr(rows, cols, d[0], d[1], d[2])
    y = torch.zeros(rows, dtype=torch.float32, device=dev)
    gold = oracle.spmv_f64(rows, cols, rowptr, colind, val, x, None, 1.0, 0.0)
    out = {"config": {"workload": "c1_reference_generator_4096x4096_16_per_row", "rows": rows, "cols": cols,
                      "nnz": nnz, "alpha": 1.0, "beta": 0.0, "seed": 42},
           "unit": "us per call", "dtype": "f32",
           "note": "latency-bound (0.8 MB of operands): no roofline figure is claimed for it"}
    for name, pre in (("prepared", True), ("unprepared", False)):
        op = osa.SpmvOp(handle, csr, osa.DnVec(d[3]), osa.DnVec(y), preprocess=pre)
        y.fill_(float("nan"))
        op(1.0, 0.0)
        stream.synchronize()
        err = oracle.max_rel_err(y.cpu().numpy(), gold)
        if err > 1e-5:
            sys.exit("bench.py: c1 (%s) differs from the fp64 oracle (%.3g)" % (name, err))
        for _ in range(200):
            op(1.0, 0.0)
        stream.synchronize()
        ms, ms_min, _, nrounds, spread = time_rounds(torch, stream, lambda i: op(1.0, 0.0), 100, None, 20.0)
        # one call at a time: launch, then wait for it (what a caller that needs y at once sees)
        t0 = time.perf_counter()
        for _ in range(200):
            op(1.0, 0.0)
            stream.synchronize()
        sync_us = (time.perf_counter() - t0) / 200 * 1e6
        out[name] = {"us_per_call_back_to_back": round(ms * 1e3, 3), "us_per_call_fastest_round": round(ms_min * 1e3, 3),
                     "us_per_call_with_synchronize": round(sync_us, 2), "rounds": nrounds,
                     "gflops_back_to_back": round(2.0 * nnz / (ms * 1e-3) / 1e9, 2),
                     "gpu_vs_fp64_oracle_max_rel_err": err}
    oracle.spmv_f32(rows, rowptr, colind, val, x, np.zeros(rows, np.float32), 1.0, 0.0)
    t0 = time.perf_counter()
    reps = 2000
    for _ in range(reps):
        oracle.spmv_f32(rows, rowptr, colind, val, x, np.zeros(rows, np.float32), 1.0, 0.0)
    dt = (time.perf_counter() - t0) / reps
    out["cpu_baseline"] = {"value": round(dt * 1e6, 2), "unit": "us per call", "cores": 1, "kind": "port",
                           "gflops": round(2.0 * nnz / dt / 1e9, 3),
                           "sample": "%d repeats of the reference's SpmvCpu loop restated in oracle/oracle.c on the "
                                     "whole matrix (through ctypes, a fresh y each)" % reps}
    log("c1        prepared %.2f us, unprepared %.2f us per call back to back; SpmvCpu %.1f us"
        % (out["prepared"]["us_per_call_back_to_back"], out["unprepared"]["us_per_call_back_to_back"], dt * 1e6))
    return out


def run_shapes(args, osa, wl, torch, dev, stream, handle):
    """Time per call on the secondary shapes that the selection thresholds were set from: which plan a matrix gets
    (the layouts from 7 M entries, 31 % / 19 % far gathers, 2^18 columns; the long-row cut-offs) is decided by these
    grids.  Per shape: the default plan as selected, the default plan forced onto the caller's arrays (merge path /
    row-wise kernels), the default plan with repeatable sums, and ACL_SPARSE_SPMV_CSR_ALG2.  --scale below 1 keeps
    the first shapes of every group only."""
    i64 = torch.int64

    def rows_of(rows, per_row, cols, seed, sort):
        """`per_row` random columns a row, unsorted (repeats possible) or sorted."""
        idx = torch.arange(rows * per_row, dtype=i64, device=dev)
        ci = (wl._lsr(wl.hash64(seed, idx), 11) % cols).view(rows, per_row)
        if sort:
            ci = ci.sort(dim=1).values
        return {"rows": rows, "cols": cols, "rowptr": (torch.arange(rows + 1, dtype=i64, device=dev) * per_row).int(),
                "colind": ci.reshape(-1).int(), "values": wl.uniform(seed + 1, rows * per_row, -1.0, 1.0, dev)}

    def band(rows, near, far, seed):
        idx = torch.arange(rows * (near + far), dtype=i64, device=dev)
        h = wl._lsr(wl.hash64(seed, idx), 11).view(rows, near + far)
        r = torch.arange(rows, dtype=i64, device=dev).view(rows, 1)
        ci = torch.cat([(r + h[:, :near] % 81 - 40).clamp(0, rows - 1), h[:, near:] % rows], dim=1).sort(dim=1).values
        return {"rows": rows, "cols": rows, "colind": ci.reshape(-1).int(),
                "rowptr": (torch.arange(rows + 1, dtype=i64, device=dev) * (near + far)).int(),
                "values": wl.uniform(seed + 1, rows * (near + far), -1.0, 1.0, dev)}

    def power_law(m, alpha, lmax, mean):
        A = wl.power_law_csr(m, m, alpha, 1, lmax, 2001, dev, target_mean=mean)
        A["values"] = wl.uniform(2002, A["colind"].numel(), -1.0, 1.0, dev)
        return A

    M = 1 << 20
    groups = {
        "equal_rows_unsorted_columns": [("%g M x %d (%g M columns)" % (r / 1e6, k, c / 1e6),
                                         lambda r=r, k=k, c=c: rows_of(r, k, c, 7, False))
                                        for r, k, c in ((1000000, 4, 1100000), (1500000, 4, 1600000),
                                                        (2000000, 4, 2200000), (1000000, 8, 2200000),
                                                        (3000000, 3, 8000000), (2000000, 8, 2200000),
                                                        (6000000, 2, 20000000), (2000000, 8, 33000000),
                                                        (4000000, 4, 33000000), (1000000, 32, 16000000),
                                                        (4000000, 8, 16000000), (2000000, 16, 30000000),
                                                        (16000000, 2, 16000000), (8000000, 4, 33000000))],
        "band_plus_random_4M_rows": [("%d + %d" % (n, f), lambda n=n, f=f: band(4000000, n, f, 11))
                                     for n, f in ((5, 1), (15, 1), (14, 2), (12, 4), (4, 4), (30, 2), (30, 6), (60, 4))],
        "equal_rows_sorted_columns": [("%d x %d (x of %g M)" % (r, k, c / 1e6),
                                       lambda r=r, k=k, c=c: rows_of(r, k, c, 13, True))
                                      for c in (3000000, 8000000, 300000, 600000, 1000000)
                                      for r, k in ((20000, 2000), (50000, 1100), (4000, 8000), (2000, 20000),
                                                   (200000, 300), (3000000, 12))
                                      if (c == 8000000) == ((r, k) == (20000, 2000)) or c < 3000000],
        "power_law": [("%g M rows, exponent %g, longest %d" % (m / M, a, lmax),
                       lambda m=m, a=a, lmax=lmax, mean=mean: power_law(m, a, lmax, mean))
                      for m, a, lmax, mean in ((1 * M, 2.0, 200000, None), (2 * M, 2.0, 200000, None),
                                               (4 * M, 2.0, 200000, None), (8 * M, 2.5, 200000, 8.0),
                                               (4 * M, 1.6, 100000, None))],
    }
    plans = (("default", {}, 0), ("default_on_callers_arrays", {"OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ": str(1 << 62)}, 0),
             ("default_repeatable", {"OPS_SPARSE_SPMV_REPEATABLE": "1"}, 0),
             ("alg2", {}, osa.ACL_SPARSE_SPMV_CSR_ALG2))
    res = {}
    for gname, shapes in groups.items():
        res[gname] = {}
        if args.scale < 1.0:
            shapes = shapes[:2]
        for sname, make in shapes:
            torch.cuda.empty_cache()
            A = make()
            rows, cols, nnz = A["rows"], A["cols"], int(A["colind"].numel())
            csr = osa.Csr(rows, cols, A["rowptr"], A["colind"], A["values"])
            x = wl.uniform(5, cols, -1.0, 1.0, dev)
            y = torch.zeros(rows, dtype=torch.float32, device=dev)
            line = {"nnz": nnz}
            for pname, env, alg in plans:
                for name in BENCH_ENV + ("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ",):
                    os.environ.pop(name, None)
                os.environ.update(env)
                op = osa.SpmvOp(handle, csr, osa.DnVec(x), osa.DnVec(y), alg=alg)
                for _ in range(3):
                    op(1.0, 0.0)
                stream.synchronize()
                ms, _, _, _, _ = time_rounds(torch, stream, lambda i: op(1.0, 0.0), 5, None, 15.0)
                line[pname] = round(ms * 1e3, 1)
                line[pname + "_buffer_mib"] = round(op.buffer.numel() / 2.0 ** 20, 1)
                del op
            for name in BENCH_ENV + ("OPS_SPARSE_DEFAULT_BLOCKED_MIN_NNZ",):
                os.environ.pop(name, None)
            res[gname][sname] = line
            log("%-28s %-40s %s" % (gname, sname, json.dumps(line)))
            del A, csr, x, y
    return res


def run_stencils(args, osa, wl, torch, dev, stream, handle):
    """The headline kernel family on other meshes and bands than c2's: time of a call (default algorithm after
    Preprocess, alpha = 1, beta = 0.5, every launch on the same operands) and the algorithmic bytes against 8 TB/s.
    What separates these shapes is the number of gathers a row needs and how many of them a cache line serves."""
    import itertools

    def band(rows, width, seed):
        """`width` distinct columns a row inside a window of 4 x width columns round the diagonal."""
        idx = torch.arange(rows * width, dtype=torch.int64, device=dev).view(rows, width)
        r = torch.arange(rows, dtype=torch.int64, device=dev).view(rows, 1)
        step = (wl._lsr(wl.hash64(seed, idx.reshape(-1)), 11) % 4).view(rows, width)
        ci = (r - 2 * width + 4 * torch.arange(width, dtype=torch.int64, device=dev).view(1, width) + step)
        ci = ci.clamp(0, rows - 1)
        return {"rows": rows, "cols": rows, "colind": ci.reshape(-1).int(),
                "rowptr": (torch.arange(rows + 1, dtype=torch.int64, device=dev) * width).int(),
                "values": wl.uniform(seed + 1, rows * width, -1.0, 1.0, dev)}

    box3 = list(itertools.product((-1, 0, 1), repeat=3))
    cross3 = [o for o in box3 if sum(abs(v) for v in o) <= 1]
    box2 = list(itertools.product((-1, 0, 1), repeat=2))
    cross2 = [o for o in box2 if sum(abs(v) for v in o) <= 1]
    shapes = [
        ("5-point, 2048^2 (c2)", lambda: wl.stencil_csr((2048, 2048), cross2, dev)),
        ("9-point, 2048^2", lambda: wl.stencil_csr((2048, 2048), box2, dev)),
        ("7-point, 160^3", lambda: wl.stencil_csr((160, 160, 160), cross3, dev)),
        ("27-point, 128^3", lambda: wl.stencil_csr((128, 128, 128), box3, dev)),
        ("band of 50, 1 M rows", lambda: band(1 << 20, 50, 21)),
        ("band of 200, 256 K rows", lambda: band(1 << 18, 200, 22)),
        ("band of 600, 64 K rows", lambda: band(1 << 16, 600, 23)),
    ]
    if args.scale < 1.0:
        shapes = shapes[:2]
    res = {}
    for name, make in shapes:
        torch.cuda.empty_cache()
        A = make()
        rows, nnz = A["rows"], int(A["colind"].numel())
        csr = osa.Csr(rows, rows, A["rowptr"], A["colind"], A["values"])
        x = wl.uniform(5, rows, -1.0, 1.0, dev)
        y0 = wl.uniform(6, rows, -1.0, 1.0, dev)
        y = y0.clone()
        op = osa.SpmvOp(handle, csr, osa.DnVec(x), osa.DnVec(y))
        for _ in range(5 + args.settle):   # (the clocks' ramp and the runtime's one-off stall: see run_workload)
            op(1.0, 0.5)
        stream.synchronize()
        ms, ms_min, _, nrounds, _ = time_rounds(torch, stream, lambda i: op(1.0, 0.5), args.steps,
                                                lambda: y.copy_(y0), args.min_gpu_ms)
        bytes_alg = wl.spmv_bytes_alg(rows, rows, nnz, 4, 4, 4, True)
        line = {"rows": rows, "nnz": nnz, "entries_per_row": round(nnz / rows, 1), "us_per_call": round(ms * 1e3, 2),
                "us_fastest_round": round(ms_min * 1e3, 2), "rounds": nrounds, "bytes_alg": bytes_alg,
                "frac_of_8TBs": round(bytes_alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
        res[name] = line
        log("%-26s %s" % (name, json.dumps(line)))
        del op, csr, A, x, y, y0
    return res


def run_spmm_shapes(args, osa, wl, torch, dev, stream, handle):
    """SpMM fp32 with 16 - 128 columns of B on meshes, bands and uniformly random columns: the two kernels a matrix
    without long rows can take - slabs staged through LDS (`OPS_SPARSE_SPMM_NO_ROWS_RULE=1` at Preprocess), a lane
    group a row straight from memory (`OPS_SPARSE_SPMM_NO_SLAB=1` at the call) - and what Preprocess picks by
    itself.  The grid behind that rule."""
    import itertools

    def band(rows, width, seed):
        idx = torch.arange(rows * width, dtype=torch.int64, device=dev).view(rows, width)
        r = torch.arange(rows, dtype=torch.int64, device=dev).view(rows, 1)
        step = (wl._lsr(wl.hash64(seed, idx.reshape(-1)), 11) % 4).view(rows, width)
        ci = (r - 2 * width + 4 * torch.arange(width, dtype=torch.int64, device=dev).view(1, width) + step)
        return {"rows": rows, "cols": rows, "colind": ci.clamp(0, rows - 1).reshape(-1).int(),
                "rowptr": (torch.arange(rows + 1, dtype=torch.int64, device=dev) * width).int(),
                "values": wl.uniform(seed + 1, rows * width, -1.0, 1.0, dev)}

    box3 = list(itertools.product((-1, 0, 1), repeat=3))
    cross3 = [o for o in box3 if sum(abs(v) for v in o) <= 1]
    shapes = [
        ("5-point, 1448^2", lambda: wl.laplacian_2d(1448, dev)),
        ("7-point, 128^3", lambda: wl.stencil_csr((128, 128, 128), cross3, dev)),
        ("27-point, 100^3", lambda: wl.stencil_csr((100, 100, 100), box3, dev)),
        ("band of 50, 256 K rows", lambda: band(1 << 18, 50, 21)),
        ("band of 200, 64 K rows", lambda: band(1 << 16, 200, 22)),
        ("8 random columns a row, 1 M rows", lambda: wl.uniform_rows_csr(1 << 20, 1 << 20, 8, 5, dev)),
        ("32 random columns a row, 512 K rows", lambda: wl.uniform_rows_csr(1 << 19, 1 << 19, 32, 7, dev)),
    ]
    if args.scale < 1.0:
        shapes = shapes[:1]
    res = {}
    for name, make in shapes:
        torch.cuda.empty_cache()
        A = make()
        rows, nnz = A["rows"], int(A["colind"].numel())
        csr = osa.Csr(rows, A["cols"], A["rowptr"], A["colind"], A["values"])
        res[name] = {"rows": rows, "nnz": nnz, "widths": {}}
        for n in (16, 32, 64, 128):
            B = wl.uniform(7, A["cols"] * n, -1.0, 1.0, dev)
            C = torch.zeros(rows * n, dtype=torch.float32, device=dev)
            dB, dC = osa.DnMat(A["cols"], n, n, B), osa.DnMat(rows, n, n, C)

            def timed(op):
                for _ in range(10):
                    op(1.0, 0.0)
                stream.synchronize()
                return round(time_rounds(torch, stream, lambda i: op(1.0, 0.0), args.steps, None,
                                         min(args.min_gpu_ms, 20.0))[0] * 1e3, 1)

            line = {"picked_us": timed(osa.SpmmOp(handle, csr, dB, dC))}
            os.environ["OPS_SPARSE_SPMM_NO_ROWS_RULE"] = "1"
            slabs = osa.SpmmOp(handle, csr, dB, dC)
            del os.environ["OPS_SPARSE_SPMM_NO_ROWS_RULE"]
            line["slabs_us"] = timed(slabs)
            os.environ["OPS_SPARSE_SPMM_NO_SLAB"] = "1"
            line["rows_us"] = timed(slabs)
            del os.environ["OPS_SPARSE_SPMM_NO_SLAB"]
            bytes_alg = wl.spmm_bytes_alg(rows, A["cols"], n, nnz, 4, 4, 4, False)
            line["frac_of_8TBs"] = round(bytes_alg / (line["picked_us"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)
            res[name]["widths"]["n=%d" % n] = line
            log("%-36s n=%-4d %s" % (name, n, json.dumps(line)))
            del slabs, B, C, dB, dC
        del csr, A
    return res


def run_few_columns(args, osa, wl, torch, dev, stream, handle):
    """SpMM with one to sixteen columns of B (a few right-hand sides, block Krylov methods) on meshes: time of a
    call after Preprocess (alpha = 1, beta = 0), the algorithmic bytes against 8 TB/s, the same product as n
    SpMV calls, and the call with the kernel for narrow B switched off (the lane-group kernels it replaced)."""
    import itertools
    box3 = list(itertools.product((-1, 0, 1), repeat=3))
    cross3 = [o for o in box3 if sum(abs(v) for v in o) <= 1]
    cross2 = [(-1, 0), (0, -1), (0, 0), (0, 1), (1, 0)]
    shapes = [
        ("5-point, 2048^2 (c2)", lambda: wl.stencil_csr((2048, 2048), cross2, dev)),
        ("7-point, 160^3", lambda: wl.stencil_csr((160, 160, 160), cross3, dev)),
        ("27-point, 128^3", lambda: wl.stencil_csr((128, 128, 128), box3, dev)),
    ]
    if args.scale < 1.0:
        shapes = shapes[:1]
    cases = [(torch.float32, n, order) for n in (1, 2, 4, 8) for order in ("row", "col")]
    cases += [(torch.float16, 8, "row"), (torch.float16, 16, "row")]
    res = {}
    for name, make in shapes:
        torch.cuda.empty_cache()
        A = make()
        rows, nnz = A["rows"], int(A["colind"].numel())
        x = wl.uniform(5, rows, -1.0, 1.0, dev)
        y = torch.zeros(rows, dtype=torch.float32, device=dev)
        csr32 = osa.Csr(rows, rows, A["rowptr"], A["colind"], A["values"])
        sv = osa.SpmvOp(handle, csr32, osa.DnVec(x), osa.DnVec(y))
        for _ in range(5 + args.settle):   # (the clocks' ramp and the runtime's one-off stall: see run_workload)
            sv(1.0, 0.0)
        stream.synchronize()
        spmv_us = time_rounds(torch, stream, lambda i: sv(1.0, 0.0), args.steps, None, args.min_gpu_ms)[0] * 1e3
        res[name] = {"rows": rows, "nnz": nnz, "spmv_us": round(spmv_us, 2), "cases": {}}
        log("%s: SpMV %.1f us" % (name, spmv_us))
        for dtype, n, order in cases:
            vb = 4 if dtype == torch.float32 else 2
            vals = A["values"].to(dtype)
            csr = osa.Csr(rows, rows, A["rowptr"], A["colind"], vals)
            B = wl.uniform(7, rows * n, -1.0, 1.0, dev).to(dtype)
            C = torch.zeros(rows * n, dtype=torch.float32, device=dev)
            if order == "row":
                dB, dC = osa.DnMat(rows, n, n, B), osa.DnMat(rows, n, n, C)
            else:
                dB = osa.DnMat(rows, n, rows, B, osa.ACL_SPARSE_ORDER_COL)
                dC = osa.DnMat(rows, n, rows, C, osa.ACL_SPARSE_ORDER_COL)
            op = osa.SpmmOp(handle, csr, dB, dC)
            line = {}
            for label, env in (("us_per_call", None), ("us_without_the_narrow_kernel", "OPS_SPARSE_SPMM_NO_NARROW")):
                if env is not None:
                    os.environ[env] = "1"
                for _ in range(5):
                    op(1.0, 0.0)
                stream.synchronize()
                ms = time_rounds(torch, stream, lambda i: op(1.0, 0.0), args.steps, None, args.min_gpu_ms)[0]
                line[label] = round(ms * 1e3, 2)
                if env is not None:
                    del os.environ[env]
            bytes_alg = wl.spmm_bytes_alg(rows, rows, n, nnz, vb, vb, 4, False)
            line["bytes_alg"] = bytes_alg
            line["frac_of_8TBs"] = round(bytes_alg / (line["us_per_call"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)
            line["n_spmv_calls_us"] = round(n * spmv_us, 2)
            key = "%s n=%d %s-major" % ("fp32" if vb == 4 else "fp16->fp32", n, order)
            res[name]["cases"][key] = line
            log("  %-28s %s" % (key, json.dumps(line)))
            del op, csr, B, C, dB, dC
        del sv, csr32, A, x, y
    return res


def run_cache_probe(args, osa, wl, torch, dev, stream, handle):
    """What the 256 MB Infinity Cache is worth on this path.  (1) The copy and read kernels on buffers from 8 MiB
    to 1 GiB, launched back to back on the same buffer.  (2) The c4 product (1 M rows of 32 entries, n = 64,
    fp32) with the column indices drawn from the first `w` rows of B only, w x 256 bytes from 4 MiB to the whole
    256 MiB: same entries, same bytes gathered, only the footprint of the gathered rows changes."""
    L = osa.lib()
    sp = ctypes.c_void_p(stream.cuda_stream)
    res = {"yardsticks": {}, "c4_b_window": {}}
    for mib in (8, 16, 32, 64, 128, 512, 1024):
        nb = mib << 20
        src = torch.zeros(nb, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        tc = time_rounds(torch, stream, lambda i: L.opsparse_copy_launch(src.data_ptr(), dst.data_ptr(), nb, sp), 20,
                         None, 30.0)
        tr = time_rounds(torch, stream, lambda i: L.opsparse_read_launch(src.data_ptr(), nb, None, sp), 20, None, 30.0)
        res["yardsticks"]["%d_MiB" % mib] = {"copy_gbps": round(2 * nb / tc[0] / 1e6, 0),
                                             "read_gbps": round(nb / tr[0] / 1e6, 0)}
        log("buffer %4d MiB: copy %7.0f GB/s, read %7.0f GB/s" % (mib, 2 * nb / tc[0] / 1e6, nb / tr[0] / 1e6))
        del src, dst
    m, n = 1 << 20, 64
    B = wl.uniform(3002, m * n, -1.0, 1.0, dev).view(m, n)
    for wrows in (1 << 14, 1 << 15, 1 << 17, 1 << 18, 1 << 19, 1 << 20):
        A = wl.uniform_rows_csr(m, wrows, 32, 3001, dev)
        csr = osa.Csr(m, m, A["rowptr"], A["colind"], A["values"])
        C = torch.zeros(m, n, device=dev)
        op = osa.SpmmOp(handle, csr, osa.DnMat(m, n, n, B), osa.DnMat(m, n, n, C))
        op(1.0, 0.0)
        stream.synchronize()
        t = time_rounds(torch, stream, lambda i: op(1.0, 0.0), 5, None, args.min_gpu_ms)
        gathered = m * 32 * (8 + 256) + m * 256
        res["c4_b_window"]["%d_MiB" % (wrows * 256 >> 20)] = {"ms": round(t[0], 4),
                                                             "gather_model_gbps": round(gathered / t[0] / 1e6, 0)}
        log("c4 shape, columns within the first %8d rows of B (%3d MiB): %.3f ms, gather model %.2f TB/s"
            % (wrows, wrows * 256 >> 20, t[0], gathered / t[0] / 1e9))
        del op, csr, A, C
    return res


def run_convert(args, osa, torch, dev, stream, handle):
    """The CSR producers (coo2csr, csr2coo, csrsort, csr2csc, coosort) on 33.5 M and 21 M entries through the aclsparse
    entry points; one JSON line with a time and an algorithmic GB/s per operation."""
    L = osa.lib()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    res = {}
    for name, m, n, per in (("uniform32", 1 << 20, 1 << 20, 32), ("lap", 1 << 22, 1 << 22, 5)):
        m, n = max(1024, int(m * args.scale)), max(1024, int(n * args.scale))
        g = torch.Generator(device=dev)
        g.manual_seed(1)
        nnz = m * per
        rowptr = (torch.arange(m + 1, device=dev, dtype=torch.int64) * per).to(torch.int32)
        col = torch.randint(0, n, (nnz,), device=dev, dtype=torch.int32, generator=g)
        val = torch.rand(nnz, device=dev, generator=g)
        rowsOut = torch.empty(nnz, dtype=torch.int32, device=dev)
        ptr2 = torch.empty(m + 1, dtype=torch.int32, device=dev)
        size = ctypes.c_size_t(0)

        def timed(fn):
            fn()
            stream.synchronize()
            ms, ms_min, _, _, _ = time_rounds(torch, stream, lambda i: fn(), 3, None, 20.0)
            return ms

        t = timed(lambda: L.aclsparseXcsr2coo(handle.h, P(rowptr), nnz, m, P(rowsOut), 0))
        res[name + "_csr2coo"] = {"ms": round(t, 4), "gbps": round(4 * (nnz + m) / t / 1e6, 1)}
        t = timed(lambda: L.aclsparseXcoo2csr(handle.h, P(rowsOut), nnz, m, P(ptr2), 0))
        if not torch.equal(ptr2, rowptr):
            sys.exit("bench.py: coo2csr(csr2coo(rowptr)) != rowptr")
        res[name + "_coo2csr"] = {"ms": round(t, 4), "gbps": round(4 * (nnz + m) / t / 1e6, 1)}
        L.aclsparseXcsrsort_bufferSizeExt(handle.h, m, n, nnz, P(rowptr), P(col), ctypes.byref(size))
        buf = torch.empty(max(16, size.value), dtype=torch.uint8, device=dev)
        d = ctypes.c_void_p(None)
        L.aclsparseCreateMatDescr(ctypes.byref(d))
        perm = torch.arange(nnz, dtype=torch.int32, device=dev)
        c2 = col.clone()
        t = timed(lambda: L.aclsparseXcsrsort(handle.h, m, n, nnz, d, P(rowptr), P(c2), P(perm), P(buf)))
        L.aclsparseDestroyMatDescr(d)
        res[name + "_csrsort"] = {"ms": round(t, 4), "gbps": round((16 * nnz + 4 * m) / t / 1e6, 1)}
        cp = torch.empty(n + 1, dtype=torch.int32, device=dev)
        ri = torch.empty(nnz, dtype=torch.int32, device=dev)
        cv = torch.empty(nnz, device=dev)
        a = (handle.h, m, n, nnz, P(val), P(rowptr), P(col), P(cv), P(cp), P(ri), osa.ACL_FLOAT, 1, 0, 0)
        L.aclsparseCsr2cscEx2_bufferSize(*a, ctypes.byref(size))
        buf = torch.empty(max(16, size.value), dtype=torch.uint8, device=dev)
        t = timed(lambda: L.aclsparseCsr2cscEx2(*a, P(buf)))
        # a checksum of the permutation: the transposed matrix holds the same (row, col, value) triples
        chk_in = (torch.repeat_interleave(torch.arange(m, device=dev), per).double() * 3 + col.double() * 5).sum()
        colOf = torch.repeat_interleave(torch.arange(n, device=dev), (cp[1:] - cp[:-1]).long())
        chk_out = (ri.double() * 3 + colOf.double() * 5).sum()
        if chk_in.item() != chk_out.item() or not torch.all(ri[1:][colOf[1:] == colOf[:-1]] >= ri[:-1][colOf[1:] == colOf[:-1]]):
            sys.exit("bench.py: csr2csc result fails its checksum / order check")
        res[name + "_csr2csc"] = {"ms": round(t, 4), "gbps": round((16 * nnz + 4 * (m + n)) / t / 1e6, 1),
                                  "workspace_mib": size.value >> 20}
        # COO triples of the same matrix in a shuffled order, sorted by row (then column): rows, columns and P move,
        # 12 bytes an entry in and out.  Each timed call sorts a fresh copy (the copy is part of the timed call).
        shuffle = torch.randperm(nnz, device=dev, generator=g)
        r0 = torch.repeat_interleave(torch.arange(m, device=dev, dtype=torch.int32), per)[shuffle].contiguous()
        c0 = col[shuffle].contiguous()
        p0 = torch.arange(nnz, dtype=torch.int32, device=dev)
        r1, c1, p1 = torch.empty_like(r0), torch.empty_like(c0), torch.empty_like(p0)
        L.aclsparseXcoosort_bufferSizeExt(handle.h, m, n, nnz, P(r0), P(c0), ctypes.byref(size))
        buf = torch.empty(max(16, size.value), dtype=torch.uint8, device=dev)

        def coosort():
            r1.copy_(r0), c1.copy_(c0), p1.copy_(p0)
            if L.aclsparseXcoosortByRow(handle.h, m, n, nnz, P(r1), P(c1), P(p1), P(buf)) != 0:
                sys.exit("bench.py: aclsparseXcoosortByRow failed")

        copies = timed(lambda: (r1.copy_(r0), c1.copy_(c0), p1.copy_(p0)))
        t = timed(coosort) - copies
        key = r1.long() * n + c1.long()
        if not torch.all(key[1:] >= key[:-1]) or not torch.equal(r0[p1.long()], r1) or not torch.equal(c0[p1.long()], c1):
            sys.exit("bench.py: coosort result is not sorted or P does not lead back to the input")
        res[name + "_coosort_by_row"] = {"ms": round(t, 4), "gbps": round(24 * nnz / t / 1e6, 1),
                                         "workspace_mib": size.value >> 20}
        del shuffle, r0, c0, p0, r1, c1, p1, key, buf
        log(name, json.dumps({k: v for k, v in res.items() if k.startswith(name)}))
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all",
                    choices=["all", "c1", "c2", "c3", "c3_repeatable", "c3_transposed", "c4", "c5", "convert", "cache",
                             "shapes", "stencils", "few_columns", "spmm_shapes"],
                    help="all: c2 as the headline plus c1, c3 (default plan, repeatable default plan, ALG2, "
                         "transposed), c4 and c5 in `workloads`; shapes: the grid of secondary shapes behind the "
                         "selection thresholds; stencils: the headline kernels on other meshes and bands; "
                         "few_columns: SpMM with 1 - 16 columns of B on meshes; spmm_shapes: SpMM with 16 - 128 columns on meshes, "
                         "bands and random columns under either kernel")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the workload (debugging only)")
    ap.add_argument("--min-gpu-ms", type=float, default=50.0,
                    help="rounds of --steps launches are repeated until this much GPU time has been timed")
    ap.add_argument("--settle", type=int, default=400,
                    help="untimed launches after the warm-up, before the timed rounds (the runtime's one-off stalls)")
    ap.add_argument("--warm-only", action="store_true",
                    help="time every launch on one operand set also where that fits the Infinity Cache")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-preprocess", action="store_true", help="SpMV without the Preprocess buffer")
    ap.add_argument("--alg2", action="store_true",
                    help="SpMV with ACL_SPARSE_SPMV_CSR_ALG2: Preprocess re-stores the matrix (c3: blocked gather)")
    ap.add_argument("--panels", action="store_true",
                    help="like --alg2 with the blocked-gather layout switched off: column panels (c3)")
    ap.add_argument("--gather-probe", action="store_true", help="also measure random-gather rates (stderr)")
    ap.add_argument("--vendor", action="store_true",
                    help="also time the same product through rocSPARSE's generic API, as a yard-stick beside the figures")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    osa = load_package()
    osa.lib()
    wl = importlib.import_module("ops_sparse_amd.workloads")
    dev = torch.device("cuda:0")
    stream = torch.cuda.Stream(device=dev)
    torch.cuda.set_stream(stream)  # torch's fills / uploads and the library's kernels on one stream, in order
    handle = osa.Handle(stream)

    if args.workload == "cache":
        print(json.dumps({"metric": "Infinity-Cache probe", "data": "synthetic",
                          "probe": run_cache_probe(args, osa, wl, torch, dev, stream, handle)}), flush=True)
        handle.close()
        return
    if args.workload == "c1":
        print(json.dumps({"metric": "CSR SpMV fp32, time per call on the reference's CPU-runnable case",
                          "data": "synthetic", "c1": run_c1(args, osa, torch, dev, stream, handle)}), flush=True)
        handle.close()
        return
    if args.workload == "shapes":
        print(json.dumps({"metric": "CSR SpMV fp32, time per call by shape and plan", "unit": "us",
                          "data": "synthetic", "shapes": run_shapes(args, osa, wl, torch, dev, stream, handle)}),
              flush=True)
        handle.close()
        return
    if args.workload == "stencils":
        print(json.dumps({"metric": "CSR SpMV fp32 on meshes and bands, time per call and algorithmic bytes / 8 TB/s",
                          "unit": "us", "data": "synthetic",
                          "shapes": run_stencils(args, osa, wl, torch, dev, stream, handle)}), flush=True)
        handle.close()
        return
    if args.workload == "spmm_shapes":
        print(json.dumps({"metric": "CSR SpMM fp32 by matrix shape and width: the slab kernel, the row kernel and "
                                    "what Preprocess picks", "unit": "us", "data": "synthetic",
                          "shapes": run_spmm_shapes(args, osa, wl, torch, dev, stream, handle)}), flush=True)
        handle.close()
        return
    if args.workload == "few_columns":
        print(json.dumps({"metric": "CSR SpMM with few columns of B on meshes, time per call and algorithmic bytes / "
                                    "8 TB/s", "unit": "us", "data": "synthetic",
                          "shapes": run_few_columns(args, osa, wl, torch, dev, stream, handle)}), flush=True)
        handle.close()
        return
    if args.workload == "convert":
        print(json.dumps({"metric": "CSR producers, time per call", "unit": "ms", "data": "synthetic",
                          "operations": run_convert(args, osa, torch, dev, stream, handle)}), flush=True)
        handle.close()
        return

    head_key = "c2" if args.workload == "all" else args.workload
    if head_key == "c3" and (args.alg2 or args.panels):
        head_key = "c3_panels" if args.panels else "c3_alg2"
    cpu_cache = {}
    head = run_workload(args, osa, wl, torch, dev, stream, handle, head_key, cpu_cache)
    copy_gbps, read_gbps = measure_yardsticks(osa, torch, dev, stream)
    log("copy kernel %.0f GB/s, read kernel %.0f GB/s" % (copy_gbps, read_gbps))
    if args.gather_probe:
        log("random gathers, G/s: %s" % json.dumps(measure_gather(osa, torch, wl, dev, stream)))
    head["roofline"]["copy_kernel_gbps"] = round(copy_gbps, 1)
    head["roofline"]["read_kernel_gbps"] = round(read_gbps, 1)
    out = {"metric": "SpMV/SpMM GFLOP/s + achieved HBM GB/s (% of MI355X peak), CSR fp32",
           "value": head.pop("value"), "unit": head.pop("unit"), "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "ms_per_step": head.pop("ms_per_step"), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": head.pop("dtype"), "data": "synthetic"}
    out.update(head)
    if args.workload == "all":
        out["workloads"] = {}
        for key in ("c4", "c5", "c3", "c3_repeatable", "c3_alg2", "c3_transposed"):
            out["workloads"][key] = run_workload(args, osa, wl, torch, dev, stream, handle, key, cpu_cache)
        if not args.no_cpu:
            _cfg_cache.clear()
            out["workloads"]["c1"] = run_c1(args, osa, torch, dev, stream, handle)
    print(json.dumps(out), flush=True)
    handle.close()


if __name__ == "__main__":
    main()

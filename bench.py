#!/usr/bin/env python3
"""Benchmark of the CSR SpMV / SpMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3|c4|c5|c1]

A step is one aclsparseSpMV (or aclsparseSpMM) call over one synthetic matrix
whose arrays are already resident in HBM.  The default workload is c2, the
5-point 2-D Laplacian on a 2048 x 2048 grid (m = n = 4 194 304, nnz = 20 963 328,
alpha = 1, beta = 0.5), the configuration the headline metric is quoted on.
Preprocess runs once before the timed region (its time is reported separately).

Prints ONE JSON line: GFLOP/s = 2 * nnz * ncols / t as `value`, the roofline
object (algorithmic bytes / kernel time against 8 TB/s HBM) and the CPU baseline
(the reference's CPU golden loop restated in oracle/, timed on this host).
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


def cpu_baseline_spmv(cfg, y_gpu, budget_s=15.0):
    """The reference's SpmvCpu loop (oracle.spmv_f32), one thread, on the same matrix; the GPU result of one
    launch (y_gpu) is checked against the fp64-accumulated oracle on the way."""
    import oracle
    A = cfg["A"]
    rowptr, colind = A["rowptr"].cpu().numpy(), A["colind"].cpu().numpy()
    val = A["values"].cpu().float().numpy()
    x, y0 = cfg["x"].cpu().float().numpy(), cfg["y0"].cpu().float().numpy()
    rows, nnz = A["rows"], int(colind.size)
    gold = oracle.spmv_f64(rows, A["cols"], rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"])
    err = oracle.max_rel_err(y_gpu.cpu().numpy(), gold)
    if err > 1e-5:
        sys.exit("bench.py: the GPU result differs from the fp64 oracle (max relative error %.3g > 1e-5)" % err)
    oracle.spmv_f32(rows, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"])  # warm
    reps, t0 = 0, time.perf_counter()
    while reps < 10 and time.perf_counter() - t0 < budget_s:
        oracle.spmv_f32(rows, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"])
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    # the same loop with its rows shared out among all host threads (second baseline, reported beside the first)
    threads = oracle.host_threads()
    oracle.spmv_f32_threads(rows, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"], threads)
    t0 = time.perf_counter()
    for _ in range(5):
        oracle.spmv_f32_threads(rows, rowptr, colind, val, x, y0, cfg["alpha"], cfg["beta"], threads)
    dt_all = (time.perf_counter() - t0) / 5
    return {"value": 2.0 * nnz / dt / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
            "sample": "full matrix, %d repeats of the reference's SpmvCpu loop restated in oracle/oracle.c "
                      "(fp32 accumulate), %.1f ms each" % (reps, dt * 1e3),
            "all_cores": {"value": 2.0 * nnz / dt_all / 1e9, "unit": "GFLOP/s", "cores": threads,
                          "sample": "the same loop, rows shared out among %d OpenMP threads, %.1f ms each"
                                    % (threads, dt_all * 1e3)},
            "gpu_vs_fp64_oracle_max_rel_err": err}


def cpu_baseline_spmm(cfg, c_gpu, rows_sample=262144):
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=["c2", "c3", "c4", "c5"])
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the workload (debugging only)")
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

    if args.panels:
        os.environ["OPS_SPARSE_SPMV_NO_BLOCKED"] = "1"
    layout = "column_panels" if args.panels else "blocked_gather" if args.alg2 else "csr"
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

    t_gen = time.perf_counter()
    s = args.scale
    if args.workload == "c2":
        cfg = wl.config_c2(dev, grid=max(8, int(2048 * s ** 0.5)))
    elif args.workload == "c3":
        cfg = wl.config_c3(dev, m=max(1024, int(8388608 * s)), lmax=200000 if s >= 0.05 else 2000)
    elif args.workload == "c4":
        cfg = wl.config_c4(dev, m=max(1024, int(1048576 * s)))
    else:
        cfg = wl.config_c5(dev, m=max(1024, int(2097152 * s)))
    torch.cuda.synchronize()
    A = cfg["A"]
    rows, cols, nnz = A["rows"], A["cols"], int(A["colind"].numel())
    log("workload %s: rows=%d nnz=%d (generated in %.1f s)" % (cfg["name"], rows, nnz, time.perf_counter() - t_gen))

    is_spmm = "B" in cfg
    csr = osa.Csr(rows, cols, A["rowptr"], A["colind"], A["values"])
    vb = A["values"].element_size()
    t_pre = time.perf_counter()
    if not is_spmm:
        x = cfg["x"]
        y = cfg["y0"].clone()
        X, Y = osa.DnVec(x), osa.DnVec(y)
        op = osa.SpmvOp(handle, csr, X, Y, preprocess=not args.no_preprocess,
                        alg=osa.ACL_SPARSE_SPMV_CSR_ALG2 if layout != "csr" else osa.ACL_SPARSE_SPMV_ALG_DEFAULT)
        if layout == "blocked_gather" and not osa.lib().opsparse_spmv_csr_blocked_workspace_bytes(rows, cols, nnz, 0):
            layout = "column_panels" if osa.lib().opsparse_spmv_csr_panels_workspace_bytes(rows, cols, nnz) else "csr"
        ncols = 1
        bytes_alg = wl.spmv_bytes_alg(rows, cols, nnz, vb, x.element_size(), y.element_size(), cfg["beta"] != 0)
        bytes_gather = wl.spmv_bytes_gather(rows, cols, nnz, vb, x.element_size(), y.element_size(),
                                            cfg["beta"] != 0)
        dtype = "f32"
    else:
        n = cfg["n"]
        B = cfg["B"].contiguous()
        Cmat = torch.zeros(rows, n, dtype=torch.float32, device=dev)
        Bd = osa.DnMat(cols, n, n, B)
        Cd = osa.DnMat(rows, n, n, Cmat)
        op = osa.SpmmOp(handle, csr, Bd, Cd)
        ncols = n
        bytes_alg = wl.spmm_bytes_alg(rows, cols, n, nnz, vb, B.element_size(), 4, cfg["beta"] != 0)
        bytes_gather = wl.spmm_bytes_gather(rows, cols, n, nnz, vb, B.element_size(), 4, cfg["beta"] != 0)
        dtype = "f32" if vb == 4 else "f16 in, f32 accumulate/out"
    stream.synchronize()
    first_use_ms = (time.perf_counter() - t_pre) * 1e3  # includes loading the library's kernels onto the device
    # the same GetBufferSize + buffer allocation + Preprocess once more, now that the kernels are loaded: what a
    # second matrix would cost
    t_pre = time.perf_counter()
    if not is_spmm:
        op = osa.SpmvOp(handle, csr, X, Y, preprocess=not args.no_preprocess, alg=op.alg)
    else:
        op = osa.SpmmOp(handle, csr, Bd, Cd)
    stream.synchronize()
    preprocess_ms = (time.perf_counter() - t_pre) * 1e3

    alpha, beta = cfg["alpha"], cfg["beta"]
    first_result = None
    if not args.no_cpu:  # one launch from the initial y / C, kept for the check in the CPU leg
        op(alpha, beta)
        stream.synchronize()
        first_result = (y if not is_spmm else Cmat).clone()
    for _ in range(args.warmup):
        op(alpha, beta)
    stream.synchronize()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(args.steps):
        op(alpha, beta)
    e1.record(stream)
    stream.synchronize()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms = e0.elapsed_time(e1) / args.steps  # HIP events on the stream the kernels run on

    flops = 2.0 * nnz * ncols
    gflops = flops / (ms * 1e-3) / 1e9
    gbps = bytes_alg / (ms * 1e-3) / 1e9
    copy_gbps, read_gbps = measure_yardsticks(osa, torch, dev, stream)
    log("%.2f us/step (wall %.2f us), %.1f GFLOP/s, %.1f GB/s algorithmic = %.1f%% of 8 TB/s; "
        "copy kernel %.0f GB/s, read kernel %.0f GB/s"
        % (ms * 1e3, wall_ms * 1e3, gflops, gbps, 100 * gbps / HBM_PEAK_GBPS, copy_gbps, read_gbps))
    if args.gather_probe:
        log("random gathers, G/s: %s" % json.dumps(measure_gather(osa, torch, wl, dev, stream)))

    traffic = load_traffic(cfg["name"] + ("+" + layout if layout != "csr" else "")) if args.scale == 1.0 else None
    out = {
        "metric": "SpMV/SpMM GFLOP/s + achieved HBM GB/s (% of MI355X peak), CSR fp32",
        "value": round(gflops, 2), "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": cfg["name"], "rows": rows, "cols": cols, "nnz": nnz, "ncols_dense": ncols,
                   "alpha": alpha, "beta": beta, "index": "int32", "preprocess_ms": round(preprocess_ms, 3), "first_use_ms": round(first_use_ms, 3),
                   "preprocessed": not args.no_preprocess, "layout": layout},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4),
                     "traffic": traffic,
                     "traffic_gbps": round(traffic / (ms * 1e-3) / 1e9, 1) if traffic else None,
                     "bytes_alg": bytes_alg, "bytes_gather_model": bytes_gather,
                     # the dense operand counted once per use instead of once: what a row-wise kernel has to move
                     # when none of its gathers hits a cache (never the headline figure: it credits cache hits)
                     "gather_model_gbps": round(bytes_gather / (ms * 1e-3) / 1e9, 1),
                     "copy_kernel_gbps": round(copy_gbps, 1), "read_kernel_gbps": round(read_gbps, 1)},
    }
    if args.vendor:
        op(alpha, 0.0)
        stream.synchronize()
        out["vendor_yardstick"] = vendor_yardstick(torch, cfg, is_spmm, flops, bytes_alg, max(5, args.steps // 4),
                                                   stream, (y if not is_spmm else Cmat).clone())
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_spmm(cfg, first_result) if is_spmm else cpu_baseline_spmv(cfg, first_result)
    print(json.dumps(out), flush=True)
    handle.close()


if __name__ == "__main__":
    main()

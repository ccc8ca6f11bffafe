#!/usr/bin/env python3
"""Benchmark of the SMO-training / kernel-evaluation path on one MI355X.

Headline workload (`--workload c4`, the default): the 500,000 x 54, 7-class one-vs-one RBF C-SVC (gamma=1, C=3,
seed 20244), the configuration the path's speed-up target is quoted on.  A "step" is one full training pass,
`SvmModel::train` on a DataSet that exists in host memory: the reference's "all training time" window
(src/thundersvm/thundersvm-train.cpp:89-94: row assembly and upload, KernelMatrix construction, every class pair's
SMO solve, coefficient assembly; no file load, no model save).  `value` is that window in a warm process; the same
pass with the rows already resident in HBM is reported beside it (`train_seconds_rows_resident`), and the first
call of a fresh process -- the thundersvm-train executable on the workload's text file -- as `cli` (load / train /
save) and `train_seconds_cold`.

The printed JSON line also carries
  * roofline: the roofed kernel with the most device time in a training trace of the workload -- get_rows -- timed
    live with device events on its launch stream at the shape of the workload's largest problem, against the roof
    that bounds it there (few features: the bytes of the rows it writes; many: the fp64 matrix cores), with the
    fraction it reaches inside training (from a phase-profiled pass); `roofline_update_f`: the same for update_f;
  * predict: rows per second from host rows and from device-resident rows, flops per row and the fraction of the
    fp64 MFMA peak;
  * configs: the same figures for the other benchmark configurations (C1; C2 dense MFMA get_rows; C3 CSR get_rows
    with both kernels; C5 epsilon-SVR with its 200,000-row predict);
  * cpu_baseline: the CPU oracle (a port of the reference's USE_CUDA=OFF path, OpenMP) timed on this host on a
    bounded sample: a few outer SMO iterations of three class pairs of different sizes; per-iteration time is
    fitted linearly in the pair's row count and applied to every pair's outer-iteration count from the GPU run
    (the trajectories are identical).  It is an estimate and labelled so.
Only one GPU is ever used.
"""
import argparse
import gc
import json
import os
import re
import shutil
import subprocess
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

FP64_MFMA_PEAK_TFLOPS = 78.6
HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="c4", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--scale", type=float, default=1.0, help="row-count scale of the workloads (1.0 = benchmark shape)")
    ap.add_argument("--cpu-seconds", type=float, default=40.0, help="CPU time budget of the baseline sample (0 = skip)")
    ap.add_argument("--others", type=int, default=1, help="also measure the other benchmark configurations (sub-blocks)")
    ap.add_argument("--cli", type=int, default=1, help="also run the thundersvm-train executable on the workload's text file (fresh process)")
    ap.add_argument("--loader-only", action="store_true", help="only write the workload's LibSVM text and time the loader (no GPU)")
    ap.add_argument("--kernels-only", action="store_true",
                    help="only launch get_rows / update_f at the workload's shape plus a 1 GiB device copy (for rocprofv3 counter runs)")
    ap.add_argument("--predict-only", action="store_true",
                    help="only train once and predict the workload's test rows, plus a 1 GiB device copy (for rocprofv3 runs)")
    return ap.parse_args()


def event_time(fn, reps, warm=2):
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps   # ms


def largest_problem(train, params):
    """The rows of the largest binary problem of the workload (the two largest classes of a multi-class set)."""
    import numpy as np
    if params["svm_type"] != 0:
        return train
    labels, counts = np.unique(train.y, return_counts=True)
    if len(labels) <= 2:
        return train
    top = labels[np.argsort(-counts)[:2]]
    return train.rows(np.flatnonzero((train.y == top[0]) | (train.y == top[1])))


def kernel_figures(train, params):
    """Times get_rows (512 rows) and update_f (ws=1024) at the shape of the workload's largest problem, through the
    C ABI, on the current stream (torch's events see exactly that stream)."""
    import numpy as np
    import torch
    from thundersvm_amd import capi
    from thundersvm_amd.model import choose_dense, indicator_run
    train = largest_problem(train, params)
    n, d = train.n, train.n_features
    nf = d + 1
    ld = (nf + 7) // 8 * 8
    out = {}
    m = 512
    idx = torch.from_numpy(np.random.default_rng(0).permutation(n)[:m].astype(np.int32)).cuda()
    kt, gamma = params.get("kernel_type", 2), params.get("gamma", 0.0)
    # rows are stored as float for the RBF / polynomial / sigmoid kernels (their values are float-rounded by
    # definition), as double for the linear kernel: the same choice KernelMatrix makes during training
    row_type = capi.ROW_F64 if kt == 0 else capi.ROW_F32
    esz = 8 if row_type == capi.ROW_F64 else 4
    row_dtype = torch.float64 if row_type == capi.ROW_F64 else torch.float32
    ldo = (n + 7) // 8 * 8
    k_out = torch.empty((m, ldo), dtype=row_dtype, device="cuda")
    val_d, col_d, ptr_d = (torch.from_numpy(a).cuda() for a in (train.val, train.col, train.ptr))
    sd = torch.empty(n, dtype=torch.float64, device="cuda")
    capi.call("tsvm_csr_self_dot", val_d.data_ptr(), ptr_d.data_ptr(), n, sd.data_ptr(), None)
    if choose_dense(n, nf, train.nnz):
        x = torch.empty((n, ld), dtype=torch.float64, device="cuda")
        capi.call("tsvm_csr_to_dense", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), n, x.data_ptr(), ld, None)
        counts = torch.empty(2 * nf, dtype=torch.int32, device="cuda")
        capi.call("tsvm_column_stats_dense", x.data_ptr(), ld, n, nf, counts.data_ptr(), None)
        stats = counts.cpu().numpy()
        first = indicator_run(stats, nf)
        masks, max_ones = None, 0
        if first < nf:
            masks = torch.empty(n, dtype=torch.int64, device="cuda")
            mo = torch.zeros(1, dtype=torch.int32, device="cuda")
            capi.call("tsvm_indicator_masks", x.data_ptr(), ld, n, first, nf - first, masks.data_ptr(), mo.data_ptr(), None)
            max_ones = int(mo.cpu()[0])
            if not indicator_run(stats, nf, max_ones)[1]:     # the rule KernelMatrix applies
                masks = None
        if masks is not None:
            run = lambda: capi.call("tsvm_get_rows_dense_indicator", x.data_ptr(), ld, None, n, first, sd.data_ptr(), masks.data_ptr(),
                                    x.data_ptr(), ld, idx.data_ptr(), m, None, sd.data_ptr(), masks.data_ptr(), max_ones, kt, gamma,
                                    0.0, 3, k_out.data_ptr(), row_type, None, ldo, None)
            name = "get_rows_dense_stream_kernel (fp64 MFMA on %d columns + %d indicator columns in the epilogue)" % (first - 1, nf - first)
            mfma_cols = first
        else:
            run = lambda: capi.call("tsvm_get_rows_dense", x.data_ptr(), ld, None, n, nf, sd.data_ptr(), x.data_ptr(), ld,
                                    idx.data_ptr(), m, sd.data_ptr(), kt, gamma, 0.0, 3, k_out.data_ptr(), row_type, None, ldo, None)
            name = "get_rows_dense_stream_kernel (fp64 MFMA)" if nf <= 128 else "get_rows_dense_kernel (fp64 MFMA)"
            mfma_cols = nf
        ms = event_time(run, 20)
        flops = 2.0 * m * n * d                                   # algorithmic: every feature column, no padding
        min_bytes = 8.0 * (m * d + n * d) + esz * m * n           # rows in, rows out
        out["get_rows"] = dict(kernel=name, ms=ms, m=m, n=n, d=d, tflops=flops / ms / 1e9,
                               frac_mfma_peak=flops / ms / 1e9 / FP64_MFMA_PEAK_TFLOPS,
                               executed_mfma_tflops=2.0 * m * n * ((mfma_cols + 3) // 4 * 4) / ms / 1e9,
                               useful_tflops=2.0 * m * train.nnz / ms / 1e9, row_bytes_per_value=esz,
                               min_bytes=min_bytes, gbs=min_bytes / ms / 1e6, frac_hbm_peak=min_bytes / ms / 1e6 / HBM_PEAK_GBS,
                               flop_per_byte=flops / min_bytes, mfma_columns=int(mfma_cols),
                               executed_frac_mfma_peak=2.0 * m * n * ((mfma_cols + 3) // 4 * 4) / ms / 1e9 / FP64_MFMA_PEAK_TFLOPS)
        del x
    else:
        max_nnz = int(np.diff(train.ptr).max())
        lds = capi.kernel_lib().tsvm_get_rows_csr_sliced_lds(nf, max_nnz, capi.ROW_F32)
        w = None
        if lds > 0:
            # what KernelMatrix::get_rows enqueues when the shape fits: the stored rows streamed from their sliced copy
            # (made once per matrix), the working rows as a tile in LDS
            n_slices = (n + 63) // 64
            lens = np.diff(train.ptr)
            widths = np.array([lens[s * 64:(s + 1) * 64].max(initial=0) for s in range(n_slices)])
            sp = np.concatenate([[0], np.cumsum(64 * widths)]).astype(np.int64)
            sp_d = torch.from_numpy(sp).cuda()
            ell_col = torch.empty(int(sp[-1]), dtype=torch.int32, device="cuda")
            ell_val = torch.empty(int(sp[-1]), dtype=torch.float32, device="cuda")
            capi.call("tsvm_csr_to_sliced", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), n, sp_d.data_ptr(), nf,
                      ell_col.data_ptr(), ell_val.data_ptr(), capi.ROW_F32, None)
            run = lambda: capi.call("tsvm_get_rows_csr_sliced", ell_col.data_ptr(), ell_val.data_ptr(), capi.ROW_F32, sp_d.data_ptr(), n,
                                    sd.data_ptr(), val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), idx.data_ptr(), m, sd.data_ptr(),
                                    nf, max_nnz, kt, gamma, 0.0, 3, k_out.data_ptr(), row_type, None, ldo, None)
            kernel_name = "get_rows_csr_sliced_kernel"
            by = 8.0 * int(sp[-1]) + 8.0 * n_slices + 12.0 * lens[:m].sum() + esz * m * n      # sliced copy once, rows out
            extra = dict(sliced_entries=int(sp[-1]), passes_over_stored_rows=(m + 15) // 16)
        else:
            w = torch.zeros((nf, m), dtype=torch.float32, device="cuda")
            sdw = torch.empty(m, dtype=torch.float64, device="cuda")

            def run():
                # scatter the working rows into the (all-zero) staging matrix, the CSR kernel, take the rows out again
                capi.call("tsvm_csr_scatter_rows", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), idx.data_ptr(), m, nf,
                          w.data_ptr(), capi.ROW_F32, 0, None)
                capi.call("tsvm_gather_f64", sd.data_ptr(), idx.data_ptr(), m, sdw.data_ptr(), None)
                capi.call("tsvm_get_rows_csr_staged", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), None, n, sd.data_ptr(),
                          w.data_ptr(), capi.ROW_F32, m, sdw.data_ptr(), kt, gamma, 0.0, 3, k_out.data_ptr(), row_type, None, ldo, None)
                capi.call("tsvm_csr_scatter_rows", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), idx.data_ptr(), m, nf,
                          w.data_ptr(), capi.ROW_F32, 1, None)
            kernel_name = "get_rows_csr_kernel (+ staging scatter in and out)"
            by = 12.0 * train.nnz + 4.0 * (n + 1) + 4.0 * m * nf + esz * m * n
            extra = dict(staged_row_reads_gb=4.0 * m * train.nnz / 1e9)
        ms = event_time(run, 10)
        alg = 12.0 * train.nnz + 4.0 * (n + 1) + 4.0 * m * nf + esz * m * n      # the figure the path's roof is quoted on
        out["get_rows"] = dict(kernel=kernel_name, ms=ms, m=m, n=n, d=d, nnz=int(train.nnz),
                               gflops=2.0 * m * train.nnz / ms / 1e6, min_bytes=alg, gbs=alg / ms / 1e6,
                               frac_hbm_peak=alg / ms / 1e6 / HBM_PEAK_GBS, row_bytes_per_value=esz, bytes_this_layout=by, **extra)
        del w
    del k_out
    ws = 1024
    k_rows = torch.rand((ws, ldo), dtype=row_dtype, device="cuda")
    f = torch.zeros(n, dtype=torch.float64, device="cuda")
    ad = torch.randn(ws, dtype=torch.float64, device="cuda")
    ms = event_time(lambda: capi.call("tsvm_update_f", f.data_ptr(), ad.data_ptr(), ws, k_rows.data_ptr(), row_type, None,
                                      ldo, n, 1, None), 20)
    by = float(esz) * ws * n + 16.0 * n + 8.0 * ws   # bytes this kernel has to move with rows of esz-byte values
    out["update_f"] = dict(kernel="update_f_kernel", ms=ms, ws=ws, n=n, row_bytes_per_value=esz, min_bytes=by, gbs=by / ms / 1e6,
                           frac_hbm_peak=by / ms / 1e6 / HBM_PEAK_GBS)
    return out


def profiled_traffic(workload, kernel_prefix):
    """HBM bytes per launch of a kernel as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a copy of
    known size); read from the committed counter summary of this workload, None if there is none."""
    import re
    for stem in ("get_rows_update_f_%s_counters.md", "get_rows_csr_%s_counters.md"):
        path = os.path.join(ROOT, "profiles", stem % workload)
        if not os.path.exists(path):
            continue
        for line in open(path):
            m = re.match(r"\* `(%s[^`]*)`: .* = ([0-9.]+) GB" % kernel_prefix, line)
            if m:
                return float(m.group(2)) * 1e9
    return None


def profiled_mfma_util(workload, kernel_prefix):
    """MfmaUtil (%) of a kernel from the committed rocprofv3 counter summary of this workload, None if there is none."""
    path = os.path.join(ROOT, "profiles", "get_rows_update_f_%s_counters.md" % workload)
    if not os.path.exists(path):
        return None
    for line in open(path):
        cells = [c.strip() for c in line.split("|")]
        if len(cells) >= 7 and cells[1].startswith("`" + kernel_prefix) and re.fullmatch(r"[0-9.]+", cells[5] or "x"):
            return float(cells[5])
    return None


def cli_flags(params):
    flags = ["-s", str(params["svm_type"]), "-t", str(params["kernel_type"]), "-c", repr(float(params["C"]))]
    if "gamma" in params:
        flags += ["-g", repr(float(params["gamma"]))]
    if "p" in params:
        flags += ["-p", repr(float(params["p"]))]
    if "epsilon" in params:
        flags += ["-e", repr(float(params["epsilon"]))]
    return flags


def cli_and_loader(w, run_cli=True, loader_threads=(1, 0)):
    """Writes the workload's training rows as LibSVM text, times the loader on one thread and on all, and runs the
    thundersvm-train executable on the file in a fresh process (first call: row arena, masked streams and code objects
    are made inside its training window).  Must run before this process touches the GPU."""
    from thundersvm_amd import data as D
    from thundersvm_amd.model import Dataset
    tmp = tempfile.mkdtemp(prefix="tsvm_bench_")
    out = {}
    try:
        path = os.path.join(tmp, "train.txt")
        t0 = time.time()
        D.save_libsvm(path, w["train"])
        size = os.path.getsize(path)
        out["file"] = dict(bytes=size, rows=w["train"].n, write_seconds=time.time() - t0)
        loader = {}
        for t in loader_threads:
            best = None
            for _ in range(2):
                t0 = time.time()
                ds = Dataset(path=path, threads=t)
                dt = time.time() - t0
                assert ds.n == w["train"].n
                del ds
                best = dt if best is None else min(best, dt)
            loader["threads_%s" % ("all" if t == 0 else t)] = dict(seconds=best, mb_per_s=size / 1e6 / best)
        loader["cores"] = host_cores()
        if "threads_1" in loader and "threads_all" in loader:
            loader["speedup"] = loader["threads_1"]["seconds"] / loader["threads_all"]["seconds"]
        out["loader"] = loader
        if run_cli:
            exe = os.path.join(ROOT, "thundersvm_amd", "bin", "thundersvm-train")
            model = os.path.join(tmp, "train.model")
            t0 = time.time()
            res = subprocess.run([exe] + cli_flags(w["params"]) + [path, model], capture_output=True, text=True, timeout=600)
            wall = time.time() - t0
            log = res.stderr + res.stdout
            if res.returncode != 0:
                out["cli"] = dict(error=log[-400:])
            else:
                grab = lambda key: float(re.search(key + r" = ([0-9.eE+-]+)", log).group(1))
                out["cli"] = dict(command="thundersvm-train " + " ".join(cli_flags(w["params"])) + " train.txt train.model",
                                  load_seconds=grab("data loading time"), train_seconds=grab("all training time"),
                                  save_seconds=grab("model saving time"), process_seconds=wall,
                                  model_bytes=os.path.getsize(model),
                                  note="fresh process: the training window holds the first allocation of the row arena, the "
                                       "creation of the CU-masked streams and the loading of the kernels' code objects; the "
                                       "executable takes 45 % of the free device memory for kernel rows (a process that trains "
                                       "once pays the arena's allocation and release once), the library nine tenths; on a device "
                                       "whose memory another process has just given back (a test run right before, say) the "
                                       "arena's allocation waits for the driver to clear it: 2.5 to 4 s more")
                if w.get("test") is not None:
                    # thundersvm-predict on the model just written and the workload's test rows as text
                    test_path, pred_path = os.path.join(tmp, "test.txt"), os.path.join(tmp, "test.predict")
                    D.save_libsvm(test_path, w["test"])
                    t0 = time.time()
                    res = subprocess.run([os.path.join(ROOT, "thundersvm_amd", "bin", "thundersvm-predict"), test_path, model, pred_path],
                                         capture_output=True, text=True, timeout=600)
                    wall = time.time() - t0
                    log = res.stderr + res.stdout
                    if res.returncode != 0:
                        out["cli_predict"] = dict(error=log[-400:])
                    else:
                        out["cli_predict"] = dict(command="thundersvm-predict test.txt train.model test.predict", rows=w["test"].n,
                                                  model_load_seconds=grab("model loading time"), data_load_seconds=grab("data loading time"),
                                                  predict_seconds=grab("prediction time"), process_seconds=wall,
                                                  note="fresh process: prediction time holds the upload of the support vectors, "
                                                       "the first allocation of the row arena and the loading of the code objects")
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return out


def host_cores():
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    return min(cores, 16)


def oracle_iterations(rows, y, f0, params, iters):
    """The first `iters` outer SMO iterations of one binary problem by the CPU oracle; seconds including the
    KernelMatrix build."""
    import numpy as np
    import oracle_lib as O
    prm = O.make_param(svm_type=params["svm_type"], kernel_type=params["kernel_type"], gamma=params.get("gamma", 0.0),
                       C_=params["C"], p=params.get("p", 0.1), epsilon=params.get("epsilon", 0.001), expf_mode=1)
    t0 = time.time()
    km = O.KernelMatrix(rows.ptr, rows.col, rows.val, prm)
    res = O.smo_solve(km, y, np.zeros(rows.n), f0, prm.epsilon, params["C"], params["C"], 1024 if rows.n >= 1024 else 512,
                      out_max_iter=iters - 1)
    return time.time() - t0, res["n_iter"]


def cpu_baseline(train, params, model, budget_s):
    """Oracle (CPU port) on this host.  Binary / regression problem: the first outer iterations of the problem, scaled
    to the GPU run's iteration count.  Multi-class: three class pairs of different sizes, seconds per outer iteration
    fitted as a + b * rows, applied to every pair's iteration count."""
    import numpy as np
    cores = host_cores()
    os.environ.setdefault("OMP_NUM_THREADS", str(cores))
    n_bin = model.n_binary
    iters_gpu = [model.stats(b)["n_iter"] for b in range(n_bin)]
    if params["svm_type"] != 0 or n_bin == 1:
        if params["svm_type"] == 0:
            labels = list(model.label)
            order = np.concatenate([np.flatnonzero(train.y == labels[0]), np.flatnonzero(train.y == labels[1])])
            rows = train.rows(order)
            y = np.where(rows.y == labels[0], 1, -1).astype(np.int32)
            f0 = -y.astype(np.float64)
        else:
            n = train.n
            rows = train.rows(np.concatenate([np.arange(n), np.arange(n)]))
            y = np.concatenate([np.ones(n), -np.ones(n)]).astype(np.int32)
            f0 = np.concatenate([params["p"] - train.y, -params["p"] - train.y])
        dt, done = oracle_iterations(rows, y, f0, params, 3)
        iters = int(min(max(3 * budget_s / max(dt, 1e-3), 4), 400, iters_gpu[0]))
        if iters > 3:
            dt, done = oracle_iterations(rows, y, f0, params, iters)
        per_iter = dt / max(done, 1)
        return dict(value=per_iter * iters_gpu[0], unit="s", cores=cores, kind="port",
                    sample="oracle/liboracle.so (OpenMP port of the reference CPU path), first %d outer SMO iterations of the "
                           "%d-row problem in %.2f s (KernelMatrix build included) = %.4f s/iteration, scaled to the %d outer "
                           "iterations of the GPU run" % (done, rows.n, dt, per_iter, iters_gpu[0]),
                    seconds_per_outer_iteration=per_iter, estimate=True)
    labels = list(model.label)
    groups = [np.flatnonzero(train.y == c) for c in labels]
    pairs = [(i, j) for i in range(len(labels)) for j in range(i + 1, len(labels))]
    sizes = np.array([len(groups[i]) + len(groups[j]) for i, j in pairs])
    by_size = np.argsort(sizes)
    picks = [int(by_size[0]), int(by_size[len(by_size) // 2]), int(by_size[-1])]
    pts, notes = [], []
    for b in picks:
        i, j = pairs[b]
        rows = train.rows(np.concatenate([groups[i], groups[j]]))
        y = np.concatenate([np.ones(len(groups[i])), -np.ones(len(groups[j]))]).astype(np.int32)
        dt, done = oracle_iterations(rows, y, -y.astype(np.float64), params, 3)
        share = budget_s * sizes[b] / sizes[picks].sum()
        iters = int(min(max(3 * share / max(dt, 1e-3), 4), 200, iters_gpu[b]))
        if iters > 3:
            dt, done = oracle_iterations(rows, y, -y.astype(np.float64), params, iters)
        pts.append((sizes[b], dt / max(done, 1)))
        notes.append("%d rows: %d iterations in %.2f s" % (sizes[b], done, dt))
    xs, ys = np.array([p[0] for p in pts], dtype=float), np.array([p[1] for p in pts])
    slope, icpt = np.polyfit(xs, ys, 1)
    per_pair = np.maximum(icpt + slope * sizes, ys.min() * sizes / xs.max())
    total = float((per_pair * np.array(iters_gpu)).sum())
    return dict(value=total, unit="s", cores=cores, kind="port",
                sample="oracle/liboracle.so (OpenMP port of the reference CPU path) on three of the %d class pairs (%s; KernelMatrix "
                       "build included); seconds per outer iteration fitted as %.4g + %.4g * rows and applied to each pair's outer-"
                       "iteration count from the GPU run (%d in all)" % (len(pairs), "; ".join(notes), icpt, slope, sum(iters_gpu)),
                estimate=True)


def measure_predict(model, test, d, nb):
    """Predicts `test` once from host memory and three times from rows resident in HBM (best of three)."""
    import numpy as np
    from thundersvm_amd.model import Dataset, choose_dense
    ds_test = Dataset(test)
    model.predict(test.rows(np.arange(min(test.n, 256))))
    t0 = time.time()
    model.predict(ds_test)
    pt = time.time() - t0
    dd_test = Dataset(test).to_device()
    model.predict(dd_test)
    ptd = []
    for _ in range(3):
        t0 = time.time()
        model.predict(dd_test)
        ptd.append(time.time() - t0)
    ptd = min(ptd)
    k = model.n_classes
    n_sv = int(model.total_sv)
    flops_row = 2.0 * n_sv * d + 2.0 * (k - 1) * n_sv
    # what has to move: the batch, the support vectors, the coefficients, the decision values (no kernel values)
    by = 8.0 * (test.n * d + n_sv * d + (k - 1) * n_sv + test.n * nb)
    return dict(rows=test.n, n_sv=n_sv, classes=k, seconds=pt, rows_per_s=test.n / pt,
                note="rows_per_s: test rows start in host memory; *_device_rows: rows resident in HBM "
                     "(Dataset.to_device), decision values copied back",
                seconds_device_rows=ptd, rows_per_s_device_rows=test.n / ptd,
                flops_per_row=flops_row, tflops=flops_row * test.n / pt / 1e12,
                frac_mfma_peak=flops_row * test.n / pt / 1e12 / FP64_MFMA_PEAK_TFLOPS,
                tflops_device_rows=flops_row * test.n / ptd / 1e12,
                frac_mfma_peak_device_rows=flops_row * test.n / ptd / 1e12 / FP64_MFMA_PEAK_TFLOPS,
                bytes=by, frac_hbm_peak=by / ptd / 1e9 / HBM_PEAK_GBS,
                kernel="tsvm_predict_dec_values_dense (kernel values reduced in registers)"
                       if choose_dense(n_sv, d + 1, model._sv_nnz) else
                       "tsvm_get_rows_csr + tsvm_sum_kernel_values")


def measure_config(name, w, steps, warmup, with_kernels=True, predict=True):
    """Trains `steps` times (after `warmup`) on device-resident rows, once more from host rows, once phase-profiled;
    predicts the test rows; times the kernels at the workload's shape."""
    import numpy as np
    import torch
    from thundersvm_amd.model import Dataset, Model, make_param
    train, test, params = w["train"], w.get("test"), w["params"]
    prm = make_param(**params)
    ds = Dataset(train).to_device()

    def one(dataset):
        m = Model(prm.svm_type)
        m.train(dataset, prm)
        return m

    for _ in range(warmup):
        one(ds)
    # the step: SvmModel::train on a DataSet that lives in host memory (rows are assembled and uploaded inside train)
    model, secs = None, []
    for _ in range(steps):
        model = None
        fresh = Dataset(train)
        torch.cuda.synchronize()
        t0 = time.time()
        model = one(fresh)
        torch.cuda.synchronize()
        secs.append(time.time() - t0)
        del fresh
    # the same pass when the rows are already resident in HBM
    res = []
    for _ in range(min(steps, 3)):
        torch.cuda.synchronize()
        t0 = time.time()
        one(ds)
        torch.cuda.synchronize()
        res.append(time.time() - t0)
    nb = model.n_binary
    st = [model.stats(b) for b in range(nb)]
    block = {"workload": "%s: %d x %d, %s" % (w["name"], train.n, train.n_features, json.dumps(params)),
             "train_seconds": sum(secs) / len(secs), "train_seconds_steps": secs, "train_seconds_rows_resident": min(res),
             "outer_iterations": int(sum(s["n_iter"] for s in st)), "inner_iterations": int(sum(s["local_iter"] for s in st)),
             "binary_problems": nb, "total_sv": int(model.total_sv),
             "rows_computed": int(sum(s["rows_computed"] for s in st)),
             "cache_hit_rate": float(sum(s["cache_hits"] for s in st)) / max(1, sum(s["cache_lookups"] for s in st))}
    # phase breakdown of one profiled pass (serial schedule, device events around each phase; not a timed step)
    pm = Model(prm.svm_type)
    pm.train(ds, prm, profile=True)
    ps = [pm.stats(b) for b in range(pm.n_binary)]
    block["phase_ms"] = {k: float(sum(s[k] for s in ps)) for k in ("ms_select", "ms_get_rows", "ms_local", "ms_update_f")}
    sizes = _problem_sizes(train, params, model)
    esz = 8 if params["kernel_type"] == 0 else 4
    d = train.n_features
    from thundersvm_amd.model import choose_dense
    if choose_dense(train.n, d + 1, train.nnz):
        rows_flops = sum(2.0 * s["rows_computed"] * n_cols * d for s, n_cols in zip(ps, sizes))
    else:
        rows_flops = sum(2.0 * s["rows_computed"] * train.nnz for s in ps)       # CSR: one multiply-add per stored non-zero
    upd_bytes = sum(float(esz) * s["update_rows"] * n_cols + s["n_iter"] * (16.0 * n_cols * (2 if params["svm_type"] in (3, 4) else 1) + 8.0 * 1024)
                    for s, n_cols in zip(ps, sizes))
    block["in_training"] = {
        "get_rows_tflops": rows_flops / max(block["phase_ms"]["ms_get_rows"], 1e-9) / 1e9,
        "update_f_gbs": upd_bytes / max(block["phase_ms"]["ms_update_f"], 1e-9) / 1e6,
        "solver_us_per_inner_iteration": 1e3 * block["phase_ms"]["ms_local"] / max(1, sum(s["local_iter"] for s in ps)),
        "note": "from one phase-profiled pass (one problem at a time, every phase timed with device events); ms_local includes the ws x ws block"}
    del pm
    if predict and test is not None:
        block["predict"] = measure_predict(model, test, d, nb)
    if with_kernels:
        block["kernels"] = kernel_figures(train, params)
    return block, model


def _problem_sizes(train, params, model):
    """Columns of a kernel row (stored rows) of every binary problem, in the model's pair order."""
    import numpy as np
    if params["svm_type"] != 0:
        return [train.n]
    labels = list(model.label)
    cnt = [int((train.y == c).sum()) for c in labels]
    return [cnt[i] + cnt[j] for i in range(len(labels)) for j in range(i + 1, len(labels))]


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); re-run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    from thundersvm_amd import data as D
    gen = {"c1": lambda s: D.workload_c1(s), "c2": lambda s: D.workload_c2(s), "c3": lambda s: D.workload_c3(s),
           "c4": lambda s: D.workload_c4(s, n_test=int(50000 * s)), "c5": lambda s: D.workload_c5(s)}
    w = gen[args.workload](args.scale)

    if args.loader_only:
        print(json.dumps(cli_and_loader(w, run_cli=False, loader_threads=(1, 2, 4, 8, 0))))
        return

    # the executable in a fresh process, and the loader: before this process has touched the GPU
    fresh = cli_and_loader(w, run_cli=True) if args.cli and not (args.kernels_only or args.predict_only) else {}

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    if args.kernels_only or args.predict_only:
        src = torch.empty(1 << 27, dtype=torch.float64, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)                      # plain copy of known size: 1 GiB read + 1 GiB written
        torch.cuda.synchronize()
        del src, dst
        if args.predict_only:
            from thundersvm_amd.model import Dataset, Model, make_param
            prm = make_param(**w["params"])
            model = Model(prm.svm_type).train(Dataset(w["train"]).to_device(), prm)
            print(json.dumps(measure_predict(model, w["test"], w["train"].n_features, model.n_binary)))
            return
        print(json.dumps(kernel_figures(w["train"], w["params"])))
        return

    # Python's cyclic collector walks every container object of the process when it runs a full collection
    # (30-40 ms here, once every few training calls): it is switched off while steps are timed.
    gc.collect()
    gc.disable()
    head, model = measure_config(args.workload, w, args.steps, args.warmup)
    gc.enable()
    dt = head["train_seconds"]

    kern = head["kernels"]
    uf, gr = kern["update_f"], kern["get_rows"]
    it = head["in_training"]
    traffic_unit = "bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled; from profiles/)"
    phases = head["phase_ms"]
    share = lambda key: phases[key] / max(sum(phases.values()), 1e-9)
    if "tflops" not in gr:
        roofline = dict(kernel=gr["kernel"], bound="hbm", achieved=gr["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=gr["frac_hbm_peak"],
                        traffic=profiled_traffic(args.workload, "get_rows_csr"), traffic_unit=traffic_unit, launch_ms=gr["ms"],
                        algorithmic="12*nnz + 4*(n+1) + 4*m*d + %d*m*n bytes per launch, m=%d n=%d nnz=%d" % (
                            gr["row_bytes_per_value"], gr["m"], gr["n"], gr["nnz"]))
    elif 2.0 * gr["d"] / 8.0 < 2 * 9.8:
        # few features (2d/8 flop per byte of a double-precision row is not far above the chip's 9.8 flop per byte):
        # the roof of get_rows is the memory traffic of the rows it writes
        roofline = dict(kernel=gr["kernel"], bound="hbm", achieved=gr["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=gr["frac_hbm_peak"],
                        traffic=profiled_traffic(args.workload, "get_rows_dense"), traffic_unit=traffic_unit, launch_ms=gr["ms"],
                        algorithmic="8*(m*d + n*d) + %d*m*n bytes per launch, m=%d n=%d d=%d" % (
                            gr["row_bytes_per_value"], gr["m"], gr["n"], gr["d"]),
                        mfma_util_percent=profiled_mfma_util(args.workload, "get_rows_dense"),
                        executed_mfma_tflops=gr["executed_mfma_tflops"], executed_frac_mfma_peak=gr["executed_frac_mfma_peak"],
                        algorithmic_tflops=gr["tflops"], algorithmic_frac_mfma_peak=gr["frac_mfma_peak"],
                        in_training_algorithmic_tflops=it["get_rows_tflops"],
                        note="the matrix cores execute %d of the %d columns; the others are indicator columns added in the epilogue" % (
                            gr["mfma_columns"], gr["d"]) if gr["mfma_columns"] < gr["d"] else None)
    else:
        roofline = dict(kernel=gr["kernel"], bound="mfma", achieved=gr["tflops"], peak=FP64_MFMA_PEAK_TFLOPS,
                        unit="TFLOP/s", frac=gr["frac_mfma_peak"], traffic=profiled_traffic(args.workload, "get_rows_dense"),
                        traffic_unit=traffic_unit, launch_ms=gr["ms"],
                        algorithmic="2*m*n*d flops per launch, m=%d n=%d d=%d" % (gr["m"], gr["n"], gr["d"]),
                        mfma_util_percent=profiled_mfma_util(args.workload, "get_rows_dense"),
                        frac_in_training=it["get_rows_tflops"] / FP64_MFMA_PEAK_TFLOPS,
                        in_training="2*rows*n*d over the get_rows time of a phase-profiled pass")
    roofline["share_of_phase_time"] = share("ms_get_rows")
    roofline_uf = dict(kernel="update_f_kernel (ws 1024 x n %d, %d-byte kernel values)" % (uf["n"], uf["row_bytes_per_value"]),
                       bound="hbm", achieved=uf["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=uf["frac_hbm_peak"],
                       traffic=profiled_traffic(args.workload, "update_f"), traffic_unit=traffic_unit, launch_ms=uf["ms"],
                       algorithmic="e*ws*n + 16*n + 8*ws bytes per launch, e=%d ws=1024 n=%d" % (uf["row_bytes_per_value"], uf["n"]),
                       frac_in_training=it["update_f_gbs"] / HBM_PEAK_GBS,
                       in_training="bytes of the rows with non-zero alpha_diff actually read, summed over a phase-profiled pass, over its update_f time",
                       share_of_phase_time=share("ms_update_f"))
    unroofed = dict(local_solver_share_of_phase_time=share("ms_local"), selection_share_of_phase_time=share("ms_select"),
                    note="shares of the summed phase times of one phase-profiled pass (one problem at a time); the local solver "
                         "is one workgroup bound by latency and has no roof")

    cpu = None
    if args.cpu_seconds > 0:
        cpu = cpu_baseline(w["train"], w["params"], model, args.cpu_seconds)
        cpu["gpu_train_seconds"] = dt
        cpu["ratio"] = cpu["value"] / dt
    del model

    configs = {}
    if args.others and args.scale == 1.0:
        gc.disable()
        for name in ("c1", "c2", "c5", "c3"):
            if name == args.workload:
                continue
            if name == "c3":
                for kern_name in ("rbf", "linear"):
                    blk, m = measure_config(name, D.workload_c3(args.scale, kernel=kern_name), 2, 1, with_kernels=kern_name == "rbf")
                    configs["c3_" + kern_name] = blk
                    del m
            else:
                blk, m = measure_config(name, gen[name](args.scale), 2, 1, with_kernels=name != "c1")
                if name in ("c1", "c2") and args.cpu_seconds > 0:
                    w2 = gen[name](args.scale)
                    blk["cpu_baseline"] = cpu_baseline(w2["train"], w2["params"], m, min(args.cpu_seconds, 12.0))
                configs[name] = blk
                del m
        gc.enable()

    cli = fresh.get("cli")
    line = {
        "metric": "smo_train_wall_clock", "value": dt, "unit": "s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic (seeded generator, float32-exact values)",
        "config": {"workload": head["workload"], "scale": args.scale, "working_set": 1024,
                   "window": "SvmModel::train on a DataSet in host memory (thundersvm-train.cpp:89-94: rows assembled and "
                             "uploaded inside), warm process; train_seconds_rows_resident: rows already in HBM; "
                             "train_seconds_cold: the same window in the first call of a fresh process"},
        "step_seconds": head["train_seconds_steps"],
        "train_seconds_rows_resident": head["train_seconds_rows_resident"],
        "train_seconds_cold": cli.get("train_seconds") if cli else None,
        "cli": cli, "cli_predict": fresh.get("cli_predict"), "loader": fresh.get("loader"), "text_file": fresh.get("file"),
        "solver": {"outer_iterations": head["outer_iterations"], "inner_iterations": head["inner_iterations"],
                   "binary_problems": head["binary_problems"], "total_sv": head["total_sv"], "phase_ms": head["phase_ms"],
                   "cache_hit_rate": head["cache_hit_rate"], "in_training": head["in_training"]},
        "roofline": roofline, "roofline_update_f": roofline_uf, "unroofed": unroofed, "cpu_baseline": cpu, "kernels": kern,
        "predict": head.get("predict"), "configs": configs,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

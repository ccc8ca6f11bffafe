#!/usr/bin/env python3
"""Benchmark of the SMO-training / kernel-evaluation path on one MI355X.

Headline workload (`--workload c4`, the default): the 500,000 x 54, 7-class one-vs-one RBF C-SVC (gamma=1, C=3,
seed 20244), the configuration the path's speed-up target is quoted on.  A "step" is one full training pass,
`SvmModel::train` on a DataSet that already exists: the reference's "all training time" window
(src/thundersvm/thundersvm-train.cpp:89-94: KernelMatrix construction + every class pair's SMO solve +
coefficient assembly, excluding file load and model save).  `value` is measured with the data rows already
resident in HBM when the timed region starts; the same pass from a DataSet that lives in host memory only (rows
assembled and uploaded inside train) is reported beside it as `train_seconds_with_upload`.

The printed JSON line also carries
  * roofline: the dominant bounded kernel of the headline workload, timed live with device events on its
    launch stream at the shape of the workload's largest problem, plus the fraction the same kernel reaches
    inside training (from a phase-profiled pass);
  * configs: the same figures for the other benchmark configurations (C2 dense MFMA get_rows, C3 CSR get_rows with
    both kernels, C5 epsilon-SVR with its 200,000-row predict): train seconds, outer / inner iterations, get_rows
    TFLOP/s or GB/s, update_f GB/s, predict rows/s;
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
import sys
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
    ap.add_argument("--kernels-only", action="store_true",
                    help="only launch get_rows / update_f at the workload's shape plus a 1 GiB device copy (for rocprofv3 counter runs)")
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
    from thundersvm_amd.host_rules import choose_dense, indicator_columns
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
        first = indicator_columns(counts.cpu().numpy(), nf)
        masks, max_ones = None, 0
        if first < nf:
            masks = torch.empty(n, dtype=torch.int64, device="cuda")
            mo = torch.zeros(1, dtype=torch.int32, device="cuda")
            capi.call("tsvm_indicator_masks", x.data_ptr(), ld, n, first, nf - first, masks.data_ptr(), mo.data_ptr(), None)
            max_ones = int(mo.cpu()[0])
            if (nf + 3) // 4 - (first + 3) // 4 < 2 + 3 * max_ones:     # the rule KernelMatrix applies
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
                               flop_per_byte=flops / min_bytes)
        del x
    else:
        w = torch.zeros((nf, m), dtype=torch.float32, device="cuda")
        sdw = torch.empty(m, dtype=torch.float64, device="cuda")

        def run():
            # what KernelMatrix::get_rows enqueues: scatter the working rows into the (all-zero) staging matrix,
            # the CSR kernel, take the rows out again
            capi.call("tsvm_csr_scatter_rows", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), idx.data_ptr(), m, nf,
                      w.data_ptr(), capi.ROW_F32, 0, None)
            capi.call("tsvm_gather_f64", sd.data_ptr(), idx.data_ptr(), m, sdw.data_ptr(), None)
            capi.call("tsvm_get_rows_csr_staged", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), None, n, sd.data_ptr(),
                      w.data_ptr(), capi.ROW_F32, m, sdw.data_ptr(), kt, gamma, 0.0, 3, k_out.data_ptr(), row_type, None, ldo, None)
            capi.call("tsvm_csr_scatter_rows", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), idx.data_ptr(), m, nf,
                      w.data_ptr(), capi.ROW_F32, 1, None)
        ms = event_time(run, 10)
        by = 12.0 * train.nnz + 4.0 * (n + 1) + 4.0 * m * nf + esz * m * n
        out["get_rows"] = dict(kernel="get_rows_csr_kernel (+ staging scatter in and out)", ms=ms, m=m, n=n, d=d, nnz=int(train.nnz),
                               gflops=2.0 * m * train.nnz / ms / 1e6, min_bytes=by, gbs=by / ms / 1e6,
                               frac_hbm_peak=by / ms / 1e6 / HBM_PEAK_GBS, row_bytes_per_value=esz,
                               staged_row_reads_gb=4.0 * m * train.nnz / 1e9)
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
    model, secs = None, []
    for _ in range(steps):
        model = None
        torch.cuda.synchronize()
        t0 = time.time()
        model = one(ds)
        torch.cuda.synchronize()
        secs.append(time.time() - t0)
    # the same pass when the DataSet only exists in host memory: rows are assembled and uploaded inside train()
    up = []
    for _ in range(2):
        fresh = Dataset(train)
        torch.cuda.synchronize()
        t0 = time.time()
        one(fresh)
        torch.cuda.synchronize()
        up.append(time.time() - t0)
        del fresh
    nb = model.n_binary
    st = [model.stats(b) for b in range(nb)]
    block = {"workload": "%s: %d x %d, %s" % (w["name"], train.n, train.n_features, json.dumps(params)),
             "train_seconds": sum(secs) / len(secs), "train_seconds_steps": secs, "train_seconds_with_upload": min(up),
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
    from thundersvm_amd.host_rules import choose_dense
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
        ds_test = Dataset(test)
        model.predict(test.rows(np.arange(min(test.n, 256))))
        t0 = time.time()
        model.predict(ds_test)
        pt = time.time() - t0
        block["predict"] = dict(rows=test.n, seconds=pt, rows_per_s=test.n / pt, n_sv=int(model.total_sv),
                                note="test rows start in host memory")
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
    import torch
    from thundersvm_amd import data as D

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    gen = {"c1": lambda s: D.workload_c1(s), "c2": lambda s: D.workload_c2(s), "c3": lambda s: D.workload_c3(s),
           "c4": lambda s: D.workload_c4(s, n_test=int(50000 * s)), "c5": lambda s: D.workload_c5(s)}
    w = gen[args.workload](args.scale)

    if args.kernels_only:
        src = torch.empty(1 << 27, dtype=torch.float64, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)                      # plain copy of known size: 1 GiB read + 1 GiB written
        torch.cuda.synchronize()
        del src, dst
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
    if "tflops" not in gr:
        roofline = dict(kernel=gr["kernel"], bound="hbm", achieved=gr["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=gr["frac_hbm_peak"],
                        traffic=profiled_traffic(args.workload, "get_rows_csr"),
                        traffic_unit="bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled; from profiles/)", launch_ms=gr["ms"],
                        algorithmic="12*nnz + 4*(n+1) + 4*m*d + %d*m*n bytes per launch, m=%d n=%d nnz=%d" % (
                            gr["row_bytes_per_value"], gr["m"], gr["n"], gr["nnz"]))
    elif gr["d"] < 64:
        # few features: get_rows is bound by writing the rows, and update_f (reading them back) is the kernel with the
        # most device time among the bounded ones; both are HBM kernels
        roofline = dict(kernel="update_f_kernel (ws 1024 x n %d, %d-byte kernel values)" % (uf["n"], uf["row_bytes_per_value"]),
                        bound="hbm", achieved=uf["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=uf["frac_hbm_peak"],
                        traffic=profiled_traffic(args.workload, "update_f"),
                        traffic_unit="bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled; from profiles/)",
                        launch_ms=uf["ms"], algorithmic="e*ws*n + 16*n + 8*ws bytes per launch, e=%d ws=1024 n=%d" % (uf["row_bytes_per_value"], uf["n"]),
                        frac_in_training=it["update_f_gbs"] / HBM_PEAK_GBS,
                        in_training="bytes of the rows with non-zero alpha_diff actually read, summed over a phase-profiled pass, over its update_f time")
    else:
        roofline = dict(kernel=gr["kernel"], bound="mfma", achieved=gr["tflops"], peak=FP64_MFMA_PEAK_TFLOPS,
                        unit="TFLOP/s", frac=gr["frac_mfma_peak"], traffic=profiled_traffic(args.workload, "get_rows_dense"),
                        traffic_unit="bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled; from profiles/)",
                        launch_ms=gr["ms"], algorithmic="2*m*n*d flops per launch, m=%d n=%d d=%d" % (gr["m"], gr["n"], gr["d"]),
                        frac_in_training=it["get_rows_tflops"] / FP64_MFMA_PEAK_TFLOPS,
                        in_training="2*rows*n*d over the get_rows time of a phase-profiled pass")

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

    line = {
        "metric": "smo_train_wall_clock", "value": dt, "unit": "s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic (seeded generator, float32-exact values)",
        "config": {"workload": head["workload"], "scale": args.scale, "working_set": 1024,
                   "window": "SvmModel::train, data rows resident in HBM (thundersvm-train.cpp:89-94 without the upload; "
                             "train_seconds_with_upload has it)"},
        "step_seconds": head["train_seconds_steps"],
        "train_seconds_with_upload": head["train_seconds_with_upload"],
        "solver": {"outer_iterations": head["outer_iterations"], "inner_iterations": head["inner_iterations"],
                   "binary_problems": head["binary_problems"], "total_sv": head["total_sv"], "phase_ms": head["phase_ms"],
                   "cache_hit_rate": head["cache_hit_rate"], "in_training": head["in_training"]},
        "roofline": roofline, "cpu_baseline": cpu, "kernels": kern, "predict": head.get("predict"), "configs": configs,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

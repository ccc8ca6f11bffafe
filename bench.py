#!/usr/bin/env python3
"""Benchmark of the SMO-training / kernel-evaluation path on one MI355X.

A "step" is one full training pass (SvmModel::train: KernelMatrix construction + the SMO solve,
the reference's "all training time" window, src/thundersvm/thundersvm-train.cpp:89-94) over a fixed
synthetic workload already resident in host memory.  Default workload: C2 = binary C-SVC, RBF
(gamma=0.125, C=10) on 100,000 x 784 pixel-like rows (seed 20242).  The printed JSON line also
carries
  * roofline: the dominant kernel of that workload (dense MFMA get_rows), timed live with device
    events on the launch stream, as a fraction of the fp64 MFMA peak;
  * kernels: get_rows / update_f / predict figures for the same shape;
  * cpu_baseline: the CPU oracle (a port of the reference's USE_CUDA=OFF path, OpenMP) timed on
    this host on a bounded sample: the first `cpu_iters` outer SMO iterations of the same problem,
    scaled to the outer-iteration count of the full GPU run (the trajectories are identical).
Only one GPU is ever used.
"""
import argparse
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
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--scale", type=float, default=1.0, help="row-count scale of the workload (1.0 = benchmark shape)")
    ap.add_argument("--cpu-iters", type=int, default=-1, help="outer iterations of the CPU baseline sample (-1 = auto, 0 = skip)")
    ap.add_argument("--extra-c4", type=int, default=1, help="also time one training pass of C4 (500k x 54, 7 classes)")
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


def kernel_figures(train, params):
    """Times get_rows (512 rows) and update_f (ws=1024) at the workload's shape through the C ABI."""
    import numpy as np
    import torch
    from thundersvm_amd import capi
    n, d = train.n, train.n_features
    nf = d + 1
    ld = (nf + 7) // 8 * 8
    out = {}
    dense_ok = ld * n * 8 < 40e9 and ld <= 32 * max(train.nnz / n, 1)
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
    if dense_ok:
        x = torch.empty((n, ld), dtype=torch.float64, device="cuda")
        capi.call("tsvm_csr_to_dense", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), n, x.data_ptr(), ld, None)
        ms = event_time(lambda: capi.call("tsvm_get_rows_dense", x.data_ptr(), ld, None, n, nf, sd.data_ptr(), x.data_ptr(), ld,
                                          idx.data_ptr(), m, sd.data_ptr(), kt, gamma, 0.0, 3, k_out.data_ptr(), row_type, None, ldo,
                                          None), 20)
        flops = 2.0 * m * n * d
        out["get_rows"] = dict(kernel="get_rows_dense_kernel (fp64 MFMA)", ms=ms, m=m, n=n, d=d,
                               tflops=flops / ms / 1e9, frac_mfma_peak=flops / ms / 1e9 / FP64_MFMA_PEAK_TFLOPS,
                               useful_tflops=2.0 * m * train.nnz / ms / 1e9, row_bytes_per_value=esz,
                               write_gbs=esz * m * n / ms / 1e6)
        del x
    else:
        w = torch.empty((nf, m), dtype=torch.float64, device="cuda")
        sdw = torch.empty(m, dtype=torch.float64, device="cuda")

        def run():
            capi.call("tsvm_csr_stage_rows", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), idx.data_ptr(), m, nf,
                      w.data_ptr(), None)
            capi.call("tsvm_gather_f64", sd.data_ptr(), idx.data_ptr(), m, sdw.data_ptr(), None)
            capi.call("tsvm_get_rows_csr", val_d.data_ptr(), col_d.data_ptr(), ptr_d.data_ptr(), None, n, sd.data_ptr(),
                      w.data_ptr(), m, sdw.data_ptr(), kt, gamma, 0.0, 3, k_out.data_ptr(), row_type, None, ldo, None)
        ms = event_time(run, 10)
        by = 12.0 * train.nnz + 4.0 * (n + 1) + 8.0 * m * nf + esz * m * n
        out["get_rows"] = dict(kernel="get_rows_csr_kernel", ms=ms, m=m, n=n, d=d, gflops=2.0 * m * train.nnz / ms / 1e6,
                               gbs=by / ms / 1e6, frac_hbm_peak=by / ms / 1e6 / HBM_PEAK_GBS, row_bytes_per_value=esz)
        del w
    del k_out
    ws = 1024
    k_rows = torch.rand((ws, ldo), dtype=row_dtype, device="cuda")
    f = torch.zeros(n, dtype=torch.float64, device="cuda")
    ad = torch.randn(ws, dtype=torch.float64, device="cuda")
    ms = event_time(lambda: capi.call("tsvm_update_f", f.data_ptr(), ad.data_ptr(), ws, k_rows.data_ptr(), row_type, None,
                                      ldo, n, 1, None), 20)
    by = float(esz) * ws * n + 16.0 * n + 8.0 * ws   # bytes this kernel has to move with rows of esz-byte values
    out["update_f"] = dict(kernel="update_f_kernel", ms=ms, ws=ws, n=n, row_bytes_per_value=esz, gbs=by / ms / 1e6,
                           frac_hbm_peak=by / ms / 1e6 / HBM_PEAK_GBS)
    return out


def profiled_traffic(workload, kernel_prefix):
    """HBM bytes per launch of a kernel as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a copy of
    known size); read from the committed counter summary of this workload, None if there is none."""
    import re
    path = os.path.join(ROOT, "profiles", "get_rows_update_f_%s_counters.md" % workload)
    if not os.path.exists(path):
        return None
    for line in open(path):
        m = re.match(r"\* `(%s[^`]*)`: .* = ([0-9.]+) GB" % kernel_prefix, line)
        if m:
            return float(m.group(2)) * 1e9
    return None


def cpu_baseline(train, params, gpu_outer_iters, cpu_iters):
    """Oracle (CPU port) on this host, first `cpu_iters` outer iterations of the first binary problem."""
    import numpy as np
    import oracle_lib as O
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    cores = min(cores, 16)
    os.environ.setdefault("OMP_NUM_THREADS", str(cores))
    if params["svm_type"] == 0:
        labels = []
        for v in train.y:
            if v not in labels:
                labels.append(v)
            if len(labels) == 2:
                break
        sel = np.flatnonzero((train.y == labels[0]) | (train.y == labels[1]))
        order = np.concatenate([sel[train.y[sel] == labels[0]], sel[train.y[sel] == labels[1]]])
        sub = train.rows(order)
        y = np.where(sub.y == labels[0], 1, -1).astype(np.int32)
        f0 = -y.astype(np.float64)
        rows = sub
    else:
        n = train.n
        rows = train.rows(np.concatenate([np.arange(n), np.arange(n)]))
        y = np.concatenate([np.ones(n), -np.ones(n)]).astype(np.int32)
        f0 = np.concatenate([params["p"] - train.y, -params["p"] - train.y])
    prm = O.make_param(svm_type=params["svm_type"], kernel_type=params["kernel_type"], gamma=params.get("gamma", 0.0),
                       C_=params["C"], p=params.get("p", 0.1), epsilon=params.get("epsilon", 0.001), expf_mode=1)
    t0 = time.time()
    km = O.KernelMatrix(rows.ptr, rows.col, rows.val, prm)
    res = O.smo_solve(km, y, np.zeros(rows.n), f0, prm.epsilon, params["C"], params["C"], 1024 if rows.n >= 1024 else 512,
                      out_max_iter=cpu_iters - 1)
    dt = time.time() - t0
    done = res["n_iter"]
    return dt, done, cores, rows.n


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); re-run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    from thundersvm_amd import data as D
    from thundersvm_amd.model import Dataset, Model, make_param

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    gen = {"c1": D.workload_c1, "c2": D.workload_c2, "c3": D.workload_c3, "c4": D.workload_c4, "c5": D.workload_c5}
    w = gen[args.workload](args.scale)
    train, test, params = w["train"], w.get("test"), w["params"]
    prm = make_param(**params)

    if args.kernels_only:
        src = torch.empty(1 << 27, dtype=torch.float64, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)                      # plain copy of known size: 1 GiB read + 1 GiB written
        torch.cuda.synchronize()
        del src, dst
        print(json.dumps(kernel_figures(train, params)))
        return

    # The rows are handed to the host layer once (the reference's DataSet exists before its timed
    # model->train() call, thundersvm-train.cpp:28-29,89-94); a step is train() on that DataSet.
    ds_train = Dataset(train).to_device()   # training rows resident in HBM before the timed region
    ds_test = Dataset(test) if test is not None else None

    def one_train():
        m = Model(prm.svm_type)
        m.train(ds_train, prm)
        return m

    # Python's cyclic collector walks every container object of the process when it runs a full collection
    # (30-40 ms here, once every few training calls): it is switched off for the warm-up and timed steps.
    import gc
    gc.collect()
    gc.disable()
    for _ in range(args.warmup):
        one_train()
    # Each step is bracketed by device synchronisation on both sides.  The previous step's model (100,000 support
    # vectors held as host rows for C2) is released between the brackets: tearing a model down is not training.
    model = None
    step_seconds = []
    for _ in range(args.steps):
        model = None
        torch.cuda.synchronize()
        t0 = time.time()
        model = one_train()
        torch.cuda.synchronize()
        step_seconds.append(time.time() - t0)
    gc.enable()
    dt = sum(step_seconds) / max(args.steps, 1)
    outer = sum(model.stats(b)["n_iter"] for b in range(model.n_binary))
    inner = sum(model.stats(b)["local_iter"] for b in range(model.n_binary))
    first_outer = model.stats(0)["n_iter"]

    # phase breakdown of one profiled pass (device events around each phase; not part of the timed steps)
    pm = Model(prm.svm_type)
    pm.train(ds_train, prm, profile=True)
    phases = {k: float(sum(pm.stats(b)[k] for b in range(pm.n_binary)))
              for k in ("ms_select", "ms_get_rows", "ms_local", "ms_update_f")}
    del pm

    predict = None
    if test is not None:
        model.predict(test.rows(np.arange(min(test.n, 256))))
        t0 = time.time()
        model.predict(ds_test)
        pt = time.time() - t0
        predict = dict(rows=test.n, seconds=pt, rows_per_s=test.n / pt, n_sv=model.total_sv)

    kern = kernel_figures(train, params)
    gr = kern["get_rows"]
    if "tflops" in gr:
        roofline = dict(kernel=gr["kernel"], bound="mfma", achieved=gr["tflops"], peak=FP64_MFMA_PEAK_TFLOPS,
                        unit="TFLOP/s", frac=gr["frac_mfma_peak"], traffic=profiled_traffic(args.workload, "get_rows_dense"),
                        traffic_unit="bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled; from profiles/)",
                        launch_ms=gr["ms"],
                        algorithmic="2*m*n*d flops per launch, m=%d n=%d d=%d" % (gr["m"], gr["n"], gr["d"]))
    else:
        roofline = dict(kernel=gr["kernel"], bound="hbm", achieved=gr["gbs"], peak=HBM_PEAK_GBS, unit="GB/s",
                        frac=gr["frac_hbm_peak"], traffic=profiled_traffic(args.workload, "get_rows_csr"), launch_ms=gr["ms"],
                        algorithmic="12*nnz + 4*(n+1) + 8*m*d + %d*m*n bytes per launch" % gr["row_bytes_per_value"])

    cpu = None
    if args.cpu_iters != 0:
        iters = args.cpu_iters if args.cpu_iters > 0 else 4
        cdt, done, cores, n_sub = cpu_baseline(train, params, first_outer, iters)
        if args.cpu_iters < 0 and cdt < 8.0 and done == iters:
            iters = int(min(max(iters * 15.0 / max(cdt, 1e-3), iters + 1), 400))
            cdt, done, cores, n_sub = cpu_baseline(train, params, first_outer, iters)
        per_iter = cdt / max(done, 1)
        est = per_iter * outer if model.n_binary == 1 else None
        cpu = dict(value=est if est is not None else per_iter * first_outer, unit="s", cores=cores, kind="port",
                   sample="oracle/liboracle.so (OpenMP port of the reference CPU path), first %d outer SMO iterations of "
                          "the %d-row binary problem in %.2f s (KernelMatrix build included) = %.4f s/iteration, scaled to "
                          "the %d outer iterations the GPU run needed%s" % (
                              done, n_sub, cdt, per_iter, outer if est is not None else first_outer,
                              "" if est is not None else " for the first of %d binary problems" % model.n_binary),
                   seconds_per_outer_iteration=per_iter, gpu_seconds_per_outer_iteration=dt / max(outer, 1))

    extra = {}
    if args.extra_c4 and args.workload != "c4" and args.scale == 1.0:
        w4 = D.workload_c4(1.0)
        p4 = make_param(**w4["params"])
        ds4 = Dataset(w4["train"]).to_device()
        t0 = time.time()
        m4 = Model(0).train(ds4, p4)
        extra["c4_train_seconds"] = time.time() - t0
        extra["c4_outer_iterations"] = int(sum(m4.stats(b)["n_iter"] for b in range(m4.n_binary)))
        extra["c4_total_sv"] = int(m4.total_sv)
        del m4

    line = {
        "metric": "smo_train_wall_clock", "value": dt, "unit": "s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic (seeded generator, float32-exact values)",
        "config": {"workload": "%s: %d x %d, %s" % (w["name"], train.n, train.n_features, json.dumps(params)),
                   "scale": args.scale, "working_set": 1024},
        "step_seconds": step_seconds,
        "solver": {"outer_iterations": int(outer), "inner_iterations": int(inner), "total_sv": int(model.total_sv),
                   "phase_ms": phases},
        "roofline": roofline, "cpu_baseline": cpu, "kernels": kern, "predict": predict, "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

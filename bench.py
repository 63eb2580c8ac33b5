#!/usr/bin/env python3
"""Benchmark of the sparse_conv2d hot path on one MI355X.

A step is one pass of the sparse 1x1 convolution over one batch of synthetic
input that already lives in HBM.  The default workload is the metric
configuration: int8 activations and weights, fp32 output, N=64, 512 -> 512
channels at 14x14, 85 % unstructured zeros, per-channel scales, bias and
leaky_relu.  Prints ONE JSON line.
"""
import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
LLC_BYTES = 256 << 20  # last-level (Infinity) cache the rotation must exceed
COPY_CALIBRATION_BYTES = 64 << 20


# c3 is the headline metric; the other configurations are reported under their own names
METRICS = {
    "c1": "sparse 1x1 conv nnz-GOP/s + % HBM roofline (fp32 unstructured, N=1, 96->192@56x56, 80%)",
    "c2": "sparse 1x1 conv nnz-GOP/s + % HBM roofline (fp32 semi-structured, N=32, 256->512@28x28, 90%)",
    "c3": "sparse 1x1 conv nnz-GOP/s + % HBM roofline (int8, N=64, 512->512@14x14, 85%)",
    "c4": "sparse 1x1 conv nnz-GOP/s + % HBM roofline (int8->int8 semi-structured, N=128, 128->256@56x56, 75%)",
    "custom": "sparse 1x1 conv nnz-GOP/s + % HBM roofline (shape from the command line)",
}


def custom_case(args):
    """The case --config custom describes; sizes are bounded so that a typing mistake cannot ask for a
    tensor the box does not hold."""
    import helpers

    wl = helpers.workloads
    h, w = (1, args.N) if args.N > 0 else (args.hw, args.hw)
    if not (1 <= args.M <= 8192 and 1 <= args.K <= 8192 and 1 <= h * w <= 1 << 16 and 1 <= args.batch <= 1024 and 0.0 <= args.sparsity < 1.0):
        raise SystemExit("custom: M, K in 1..8192, positions in 1..65536, batch in 1..1024, sparsity in [0, 1)")
    if float(args.batch) * h * w * (args.M * 4 + args.K * 4) > 8e9:
        raise SystemExit("custom: more than 8 GB of input and output per launch")
    act = wl.ActivationParam() if args.act == "none" else wl.ActivationParam(args.act, Leaky_relu_alpha=0.1)
    name = "custom_%s_N%d_%dx%d_%dx%d_%s%d" % (args.kind, args.batch, args.K, args.M, h, w, "semi" if args.semi else "s", int(round(args.sparsity * 100)))
    if args.kind in ("fp32", "fp16"):
        return wl.make_fp32(name, args.batch, args.K, args.M, h, w, args.sparsity, args.semi, act, seed=args.seed)
    case = wl.make_int8(name, args.batch, args.K, args.M, h, w, args.sparsity, args.semi, act, out_int8=args.kind == "int8_int8", seed=args.seed)
    if args.kind == "int8_int8":  # three sigma of the accumulator on 127, as the MobileNet layers choose it
        sigma_acc = np_sqrt(args.K * (1.0 - args.sparsity)) * 73.3 * 73.3
        case.output_scale = float(3.0 * sigma_acc * float(case.weight_scale.mean()) * case.input_scale / 127.0)
    return case


def np_sqrt(v):
    import numpy as np

    return float(np.sqrt(v))


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--config", default="c3", choices=["c1", "c2", "c3", "c4", "c5", "calib", "mobilenet", "density-sweep", "floors", "store-shapes", "device-rates", "custom", "small-batch", "float-layers"])
    ap.add_argument("--algo", default="auto", choices=["auto", "walk", "mfma", "image"])
    ap.add_argument("--image-kernel", default="rule", choices=["rule", "regroup", "transpose", "rows"], help="which image MFMA kernel a handle uses where both apply (pl_sparse_conv_tuning.image_kernel)")
    ap.add_argument("--image-regroup", default="rule", choices=["rule", "valu"], help="regrouping image kernel: by transposing LDS reads where that exists (rule) or by the vector ALU everywhere (pl_sparse_conv_tuning.image_tr_regroup)")
    # --config custom: any shape through the same measurement (parity-checked against the oracle on two images)
    ap.add_argument("--M", type=int, default=512, help="custom: output channels")
    ap.add_argument("--K", type=int, default=512, help="custom: input channels")
    ap.add_argument("--hw", type=int, default=14, help="custom: side of the square map (H = W)")
    ap.add_argument("--N", type=int, default=0, help="custom: positions per image as a 1 x N map instead of --hw")
    ap.add_argument("--batch", type=int, default=64, help="custom: images per launch")
    ap.add_argument("--semi", action="store_true", help="custom: semi-structured mask (pairs of output channels share their nonzero columns)")
    ap.add_argument("--sparsity", type=float, default=0.85, help="custom: fraction of zero weights")
    ap.add_argument("--act", default="relu", choices=["none", "relu", "relu6", "leaky_relu", "hard_swish"], help="custom: fused activation")
    ap.add_argument("--kind", default="int8_fp32", choices=["fp32", "fp16", "int8_fp32", "int8_int8"], help="custom: input -> output precision")
    ap.add_argument("--seed", type=int, default=0, help="custom: seed of the synthetic tensors")
    ap.add_argument("--fp16", action="store_true", help="run an fp32 configuration (c1, c2) through the half-precision kernel")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-lite-program", action="store_true", help="mobilenet: skip the measurement of the C++ operator surface (a child process; left out under a profiler)")
    ap.add_argument("--cache-resident", action="store_true", help="reuse one buffer set (reported, never the headline)")
    ap.add_argument("--copy-calibration", action="store_true", help="also launch a plain 64 MiB device copy 20 times, the known-size kernel that counter runs scale FETCH_SIZE / WRITE_SIZE by")
    return ap.parse_args()


SETTLE_S = 0.06


def settle(enqueue, seconds=SETTLE_S):
    """Untimed launches until the GPU has been busy for `seconds`: the engine
    clock climbs under sustained load (the first 200 launches of the metric
    kernel average 16.9 us, later ones 10.9), and what is timed afterwards
    should not depend on how long the process has been running."""
    import torch

    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        enqueue()
        torch.cuda.synchronize()


def measured_traffic(workload, algo):
    """HBM bytes per launch from the committed counter runs (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE, scaled by a plain copy of known size); None for
    a workload that has no such run."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            t = json.load(f).get("%s/%s" % (workload, algo))
    except (OSError, ValueError):
        return None, None
    if not t:
        return None, None
    return t["read_bytes"] + t["written_bytes"], t


def cpu_baseline(case, packed, budget_s=12.0):
    """The reference's CPU path on this host: its naive test reference (the
    real header when oracle/_ref was built, else the restatement), and the
    dense per-image GEMM that Paddle-Lite's x86 conv2d 1x1 performs."""
    import numpy as np
    from oracle import oracle as O
    import helpers

    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except Exception:
        pass
    threads = int(os.environ.get("OMP_NUM_THREADS", cores))
    oc, ic = case.dense.shape
    hw = case.im_size
    ops_img = 2.0 * case.nnz * hw
    scale, bias, act = helpers.merged_for_oracle(case)
    int8 = case.dense.dtype == np.int8
    # naive path as the unit test runs it: dequantise, dense basic_gemm per image
    if int8:
        wf = O.int8_to_fp32(case.dense, 1.0)
    else:
        wf = case.dense
    use_ref = O.have_ref()
    gemm = (lambda a, b: O.ref_basic_gemm_f32(a, b, bias, act, omp=True)) if use_ref else (lambda a, b: O.basic_gemm_f32(a, b, bias, act))
    xf0 = (O.int8_to_fp32(case.x[0], 1.0) if int8 else case.x[0]).reshape(ic, hw)
    t = time.perf_counter()
    gemm(wf, xf0)
    one = time.perf_counter() - t
    del one
    n_img = 0
    t = time.perf_counter()
    while time.perf_counter() - t < budget_s:  # cycle through the batch until the budget is spent
        i = n_img % case.batch
        xf = (O.int8_to_fp32(case.x[i], 1.0) if int8 else case.x[i]).reshape(ic, hw)
        gemm(wf, xf)
        n_img += 1
    naive_s = time.perf_counter() - t
    naive = {
        "value": ops_img * n_img / naive_s / 1e9,
        "unit": "nnz-GOP/s",
        "cores": threads if use_ref else 1,
        "kind": "reference" if use_ref else "port",
        "sample": "%d images (batch of %d cycled) through the unit test's naive path (dequantise + dense basic_gemm per image, %s), %.2f s" % (n_img, case.batch, "reference header built with its own OpenMP pragmas" if use_ref else "restated, 1 thread", naive_s),
        "dense_GOPs": 2.0 * oc * ic * hw * n_img / naive_s / 1e9,
    }
    # dense per-image GEMM over the batch, all cores (port of the x86 conv2d 1x1 structure)
    kind = {helpers.capi.KIND_FP32: 0, helpers.capi.KIND_INT8_FP32: 1, helpers.capi.KIND_INT8_INT8: 2}[case.kind]
    O.dense_conv1x1(kind, case.dense, case.x[:1], scale, bias, act, threads)
    best, reps = None, 0
    t_all = time.perf_counter()
    while reps < 5 or (time.perf_counter() - t_all < 3.0 and reps < 50):
        t = time.perf_counter()
        _, used = O.dense_conv1x1(kind, case.dense, case.x, scale, bias, act, threads)
        dt = time.perf_counter() - t
        best = dt if best is None else min(best, dt)
        reps += 1
    naive["dense_port"] = {
        "value": ops_img * case.batch / best / 1e9,
        "unit": "nnz-GOP/s",
        "dense_GOPs": 2.0 * oc * ic * hw * case.batch / best / 1e9,
        "cores": used,
        "kind": "port",
        "ms": best * 1e3,
        "sample": "full batch, best of %d, exact-accumulating blocked per-image GEMM with OpenMP" % reps,
    }
    # the reference's own x86 dense conv2d 1x1 (int8 -> fp32 only: its GEMM is in-tree; the fp32 path needs
    # MKL).  Timing only: its 16-bit pair sums saturate on full-range inputs.
    if case.kind == helpers.capi.KIND_INT8_FP32 and O.have_ref_x86_gemm():
        ws = np.asarray(case.weight_scale, np.float32)
        relu = {O.ACT_RELU: (1, 1.0), O.ACT_RELU6: (2, act.relu6_coef), O.ACT_LEAKY_RELU: (3, act.leaky_alpha)}.get(act.type, (0, 1.0))
        legs = {}
        for name, th in (("serial", 1), ("all_cores", threads)):
            reps = 1
            O.ref_x86_conv1x1_s8_f32(case.x[:max(1, th)], case.dense, ws, case.input_scale, bias, relu[0], relu[1], 1, th)
            while True:
                _, secs = O.ref_x86_conv1x1_s8_f32(case.x, case.dense, ws, case.input_scale, bias, relu[0], relu[1], reps, th)
                if secs > 2.0 or reps >= 64:
                    break
                reps *= 2
            legs[name] = {"value": ops_img * case.batch * reps / secs / 1e9, "unit": "nnz-GOP/s", "dense_GOPs": 2.0 * oc * ic * hw * case.batch * reps / secs / 1e9, "cores": th, "kind": "reference",
                          "ms_per_batch": secs * 1e3 / reps,
                          "sample": "%d passes over the batch, generate_gemm_s8u8_x86_kern<float>::compute per image as Conv2dCompute<kInt8,kFloat>::Run calls it%s" % (reps, "" if th == 1 else "; images dealt to OpenMP threads (an extension: the reference's loop over images is serial)")}
        naive["x86_dense_reference"] = legs
    del packed
    return naive


def run_calib(args):
    """The precision changes either side of an int8 layer (the reference's
    calib op): fp32 -> int8 and int8 -> fp32 over a 64x128x56x56 tensor, each
    timed with HIP events over rotating buffers.  Not the headline metric:
    printed as its own JSON line."""
    import numpy as np
    import torch

    import helpers
    from oracle import oracle as O

    capi = helpers.capi
    L = capi.lib()
    n = 64 * 128 * 56 * 56
    scale = 0.0371
    n_sets = 4  # 4 x 128 MB
    rng = np.random.RandomState(0)
    xf_host = (rng.standard_normal(n) * 2.5).astype(np.float32)
    xf = [torch.from_numpy(xf_host).cuda() for _ in range(n_sets)]
    q = [torch.empty(n, dtype=torch.int8, device="cuda") for _ in range(n_sets)]
    stream = torch.cuda.current_stream().cuda_stream
    out = {}
    for name, fn, src, dst, nbytes in (("fp32_to_int8", L.pl_calib_fp32_to_int8, xf, q, 5 * n), ("int8_to_fp32", L.pl_calib_int8_to_fp32, q, xf, 5 * n)):
        def step(i):
            capi.check(fn(C.c_void_p(src[i % n_sets].data_ptr()), C.c_void_p(dst[i % n_sets].data_ptr()), n, C.c_float(scale), C.c_void_p(stream)))
        step(0)
        torch.cuda.synchronize()
        if name == "fp32_to_int8":
            assert np.array_equal(q[0][:1 << 20].cpu().numpy(), O.fp32_to_int8(xf_host[:1 << 20], scale)), "fp32_to_int8 differs from the oracle"
        else:
            assert np.array_equal(xf[0][:1 << 20].cpu().numpy(), O.int8_to_fp32(q[0][:1 << 20].cpu().numpy(), scale)), "int8_to_fp32 differs from the oracle"
        settle(lambda: [step(i) for i in range(50)])
        for i in range(args.warmup):
            step(i)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(args.steps):
            step(i)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / args.steps
        out[name] = {"kernel_us": us, "algorithmic_bytes_per_launch": nbytes, "achieved_GBs": nbytes / (us * 1e-6) / 1e9, "frac": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
    print(json.dumps({"metric": "calib fp32<->int8, 64x128x56x56", "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "data": "synthetic", "config": {"workload": "calib", "elements": n, "rotation_MB": n_sets * 5 * n / 1e6, "parity_checked": True}, "roofline": {"bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s", "kernels": out}}))
    return 0


def run_density_sweep(args):
    """Two shapes (the metric shape, and a layer with sixteen times its dense
    work for the same input and output bytes) at sparsities from 50 to 99 %,
    zeros placed at random or as whole 32x32 blocks, through every int8
    algorithm: kernel time per launch (HIP events, rotating buffers) and what
    PL_ALGO_AUTO chooses.  Every timed kernel's output is compared with the
    oracle on one image first.  Not the headline metric: printed as its own
    JSON line."""
    import numpy as np
    import torch

    import helpers

    capi, wl = helpers.capi, helpers.workloads
    L = capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    names = {capi.ALGO_ROW_WALK: "row_walk", capi.ALGO_BLOCK_MFMA: "block_mfma", capi.ALGO_IMAGE_MFMA: "image_mfma"}
    steps = max(50, min(args.steps, 300))
    rows = []
    for shape in ("metric", "wide"):
        batch, ic, oc, hw = wl.DENSITY_SHAPES[shape]
        set_bytes = batch * hw * hw * (ic + 4 * oc)
        n_sets = int(LLC_BYTES * 1.25 // set_bytes) + 1
        xs = outs = None
        for blocked in (False, True):
            for sparsity in (0.50, 0.70, 0.85, 0.90, 0.95, 0.98, 0.99):
                case = wl.config_density(shape, sparsity, blocked)
                if xs is None:
                    x0 = torch.from_numpy(case.x).cuda()
                    xs = [x0] + [x0.clone() for _ in range(n_sets - 1)]
                    outs = [torch.empty((batch, oc, hw, hw), dtype=torch.float32, device="cuda") for _ in range(n_sets)]
                    xp = (C.c_void_p * n_sets)(*[t.data_ptr() for t in xs])
                    op = (C.c_void_p * n_sets)(*[t.data_ptr() for t in outs])
                want = helpers.run_oracle(case, x=case.x[:1])
                row = {"shape": "N=%d %d->%d @%dx%d" % (batch, ic, oc, hw, hw), "sparsity": sparsity, "zeros": "blocks" if blocked else "random", "nnz": case.nnz, "kernel_us": {}}
                for a in (capi.ALGO_ROW_WALK, capi.ALGO_BLOCK_MFMA, capi.ALGO_IMAGE_MFMA, capi.ALGO_AUTO):
                    try:
                        kernel, _ = helpers.make_kernel(case, algo=a)
                    except capi.SparseConvError:
                        continue  # the shape is outside this algorithm's range
                    if a == capi.ALGO_AUTO:
                        info = kernel.info()
                        row["auto"] = names[capi.check(L.pl_sparse_conv_algo_for(kernel._handle, batch, hw * hw))]
                        row["blocks_present"] = [info["mfma_blocks"], info["mfma_blocks_total"]]
                        continue
                    capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, n_sets, batch, hw * hw, n_sets + 10, C.c_void_p(stream), None))
                    torch.cuda.synchronize()
                    assert np.array_equal(outs[0][:1].cpu().numpy(), want), "%s differs from the oracle at %s" % (names[a], row)
                    settle(lambda: capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, n_sets, batch, hw * hw, 100, C.c_void_p(stream), None)), 0.03)
                    ms = C.c_float(0.0)
                    capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, n_sets, batch, hw * hw, steps, C.c_void_p(stream), C.byref(ms)))
                    row["kernel_us"][names[a]] = round(ms.value * 1e3 / steps, 2)
                row["fastest"] = min(row["kernel_us"], key=row["kernel_us"].get)
                rows.append(row)
        del xs, outs
        torch.cuda.empty_cache()
    print(json.dumps({"metric": "int8 sparse 1x1 conv: kernel us per launch by algorithm, sparsity and zero structure", "unit": "us", "n_gpus": 1, "steps": steps, "data": "synthetic",
                      "config": {"workload": "density_sweep", "parity_checked": True}, "rows": rows}))
    return 0


# (batch, ic, oc, h, w): pointwise layers of MobileNet / ResNet / Inception kinds - channel counts on both sides of
# the limits of the tile walk's forms (271 / 543 / 1087 / 2175), maps of a multiple of 8 positions, of 4 only, and odd.
FLOAT_LAYERS = [(32, 256, 512, 28, 28), (64, 384, 384, 16, 16), (64, 512, 512, 16, 16), (64, 512, 512, 14, 14), (64, 1024, 1024, 8, 8), (64, 1024, 1024, 7, 7),
                (32, 1024, 256, 14, 14), (32, 2048, 512, 8, 8), (32, 2048, 512, 7, 7), (32, 256, 512, 27, 27), (8, 128, 256, 55, 55), (64, 192, 384, 17, 17)]


def run_float_layers(args):
    """fp32 and fp16 sparse_conv2d on layers outside the headline configurations, through the three floating-point
    walks: what the library picks (the walk with the tile and the lists in LDS on all of these), the walk over channel
    chunks and the plain walk, each forced through pl_sparse_conv_tuning.  Device time per launch (HIP events over
    400 launches, rotating buffer sets); row pairs at 70 % zeros and unstructured at 85 %.  The three walks must give
    the same bits; fp32 is also compared with the oracle on one image.  Not the headline metric: its own JSON line."""
    import numpy as np
    import torch

    import helpers

    capi, wl, pla = helpers.capi, helpers.workloads, helpers.pla
    L = capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    steps = max(50, min(args.steps, 400))
    tunings = (("library_choice", None), ("chunk_walk", capi.tuning(walk_tiled=capi.TUNE_NEVER, walk_chunked=capi.TUNE_ALWAYS)),
               ("plain_walk", capi.tuning(walk_tiled=capi.TUNE_NEVER, walk_chunked=capi.TUNE_NEVER)))
    rows = []
    for kind in ("fp32", "fp16"):
        for paired in (True, False):
            for batch, ic, oc, h, w in FLOAT_LAYERS:
                case = wl.make_fp32("layer", batch, ic, oc, h, w, 0.7 if paired else 0.85, paired, pla.ActivationParam("relu"), seed=1)
                esize, tdt = 4, torch.float32
                if kind == "fp16":
                    case.kind = capi.KIND_FP16
                    case.x = case.x.astype(np.float16)
                    esize, tdt = 2, torch.float16
                set_bytes = batch * h * w * (ic + oc) * esize
                n_sets = max(2, min(24, int(LLC_BYTES * 1.25 // set_bytes) + 1))
                x0 = torch.from_numpy(case.x).cuda()
                xs = [x0] + [x0.clone() for _ in range(n_sets - 1)]
                outs = [torch.empty((batch, oc, h, w), dtype=tdt, device="cuda") for _ in range(n_sets)]
                xp = (C.c_void_p * n_sets)(*[t.data_ptr() for t in xs])
                op = (C.c_void_p * n_sets)(*[t.data_ptr() for t in outs])
                row = {"kind": kind, "zeros": "row pairs, 70 %" if paired else "unstructured, 85 %", "shape": "N=%d %d->%d @%dx%d" % (batch, ic, oc, h, w), "kernel_us": {}}
                first = None
                for name, tune in tunings:
                    kernel, _ = helpers.make_kernel(case, force_semi=paired, tuning=tune)
                    capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, n_sets, batch, h * w, n_sets + 10, C.c_void_p(stream), None))
                    torch.cuda.synchronize()
                    got = outs[0].cpu().numpy()
                    if first is None:
                        first = got
                        if kind == "fp32":
                            want = helpers.run_oracle(case, helpers.oracle_pack(case, force_semi=paired), x=case.x[:1])
                            helpers.assert_same(case, got[:1], want, "float-layers %s" % row["shape"])
                    else:
                        assert np.array_equal(got.view(np.uint8), first.view(np.uint8)), "%s differs from the library's choice at %s" % (name, row)
                    settle(lambda: capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, n_sets, batch, h * w, 100, C.c_void_p(stream), None)), 0.03)
                    ms = C.c_float(0.0)
                    capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, n_sets, batch, h * w, steps, C.c_void_p(stream), C.byref(ms)))
                    row["kernel_us"][name] = round(ms.value * 1e3 / steps, 2)
                rows.append(row)
                del xs, outs
        torch.cuda.empty_cache()
    print(json.dumps({"metric": "floating-point sparse 1x1 conv: kernel us per launch by walk on layers outside the headline configurations", "unit": "us", "n_gpus": 1,
                      "steps": steps, "data": "synthetic", "config": {"workload": "float_layers", "parity_checked": True}, "rows": rows}))
    return 0


def load_probes():
    """bench_probes/libpl_probe.so, built on first use (hipcc) when the tree does not hold it yet."""
    import importlib

    here = os.path.dirname(os.path.abspath(__file__))
    if here not in sys.path:
        sys.path.insert(0, here)
    bp = importlib.import_module("bench_probes.build_probes")
    if not os.path.exists(bp.LIB_PATH):
        bp.build()
    return C.CDLL(bp.LIB_PATH)


def run_device_rates(args):
    """Instruction rates of a CU measured with the probes of bench_probes/rate_probes.hip: LDS reads and writes by
    width and access pattern (bytes per clock and CU), the int8 matrix instruction and the fp32 multiply-add (clocks
    per instruction and SIMD), and the launch-to-launch time of an empty grid.  One workgroup per CU; medians over
    the wavefronts of the third launch."""
    import numpy as np
    import torch

    P = load_probes()
    P.pl_probe_lds_rate.restype = C.c_int
    P.pl_probe_lds_rate.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_longlong)]
    P.pl_probe_alu_rate.restype = C.c_int
    P.pl_probe_alu_rate.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_longlong)]
    out = torch.zeros(256 * 8 * 2, dtype=torch.int64, device="cuda")
    sink = torch.zeros(16, dtype=torch.int32, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    lds_names = ["ds_read_b128, 1 KB contiguous per instruction", "ds_read_b64", "ds_read_b32", "ds_read_b64_tr_b8", "ds_write_b128", "ds_write_b64",
                 "ds_read_b128, operand cells: 16 cells per quarter wavefront, quarters 3328 B apart", "ds_read_b128, the same with quarters 3392 B apart"]
    lds = {}
    for mode, name in enumerate(lds_names):
        n = C.c_longlong(0)
        for _ in range(3):
            rc = P.pl_probe_lds_rate(mode, out.data_ptr(), sink.data_ptr(), stream, C.byref(n))
            if rc != 0:
                raise RuntimeError("pl_probe_lds_rate(%d) failed with HIP error %d" % (mode, rc))
        torch.cuda.synchronize()
        counts = out.cpu().numpy().reshape(256, 8, 2)
        wg = np.median(counts[:, :, 1].max(axis=1))  # a workgroup is through when its slowest wavefront is
        lds[name] = round(8.0 * n.value / wg, 1)
    alu_names = ["v_mfma_i32_16x16x64_i8, independent", "v_mfma_i32_16x16x64_i8, dependent chain", "v_fma_f32, independent", "4 x (v_mfma + 2 v_fma_f32): per matrix instruction"]
    alu = {}
    ticks = []
    for mode, name in enumerate(alu_names):
        for waves in (4, 8):
            n = C.c_longlong(0)
            for _ in range(3):
                rc = P.pl_probe_alu_rate(mode, waves, out.data_ptr(), sink.data_ptr(), stream, C.byref(n))
                if rc != 0:
                    raise RuntimeError("pl_probe_alu_rate(%d) failed with HIP error %d" % (mode, rc))
            torch.cuda.synchronize()
            counts = out.cpu().numpy()[:256 * waves * 2].reshape(256 * waves, 2)
            clk, ns = float(np.median(counts[:, 0])), float(np.median(counts[:, 1])) * 10.0
            per_simd = waves // 4
            alu["%s, %d wavefront%s per SIMD" % (name, per_simd, "s" if per_simd > 1 else "")] = {"clocks_per_instruction_and_SIMD": round(clk / (n.value * per_simd), 2),
                                                                                           "ns_per_instruction_and_SIMD": round(ns / (n.value * per_simd), 2)}
            ticks.append(clk / ns)
    # empty grid, launch to launch
    P.pl_probe_floor.restype = C.c_int
    P.pl_probe_floor.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_float)]
    x = torch.zeros(64 * 512 * 196, dtype=torch.int8, device="cuda")
    o = torch.zeros(64 * 512 * 196, dtype=torch.float32, device="cuda")
    xp, op = (C.c_void_p * 1)(x.data_ptr()), (C.c_void_p * 1)(o.data_ptr())
    ms = C.c_float(0.0)
    for n in (2000, 4000):
        rc = P.pl_probe_floor(0, xp, op, 1, 64, 512, 512, 196, n, stream, C.byref(ms))
        if rc != 0:
            raise RuntimeError("pl_probe_floor failed with HIP error %d" % rc)
    print(json.dumps({"metric": "instruction rates of one CU (one workgroup of eight wavefronts per CU)", "n_gpus": 1, "data": "synthetic",
                      "config": {"workload": "device_rates", "grid": "256 workgroups"},
                      "lds_bytes_per_clock_and_CU": lds, "alu": alu, "s_memtime_counts_per_ns": round(float(np.median(ticks)), 2),
                      "empty_grid_256x512_us_launch_to_launch": round(ms.value * 1e3 / 4000, 2)}))
    return 0


def run_store_shapes(args):
    """How the shape of a store instruction decides the write rate of the metric shape's fp32 output
    (64 x 512 x 14 x 14 floats, 25.7 MB; rows of 784 bytes start 16 bytes further into a 64-byte sector
    each): store-only kernels on the image kernels' grid and row assignment, rotating buffers."""
    import torch

    P = load_probes()
    P.pl_probe_store_shape.restype = C.c_int
    P.pl_probe_store_shape.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_float)]
    out_bytes = 64 * 512 * 196 * 4
    n_sets = int(LLC_BYTES * 1.25 // out_bytes) + 1
    outs = [torch.empty(out_bytes // 4, dtype=torch.float32, device="cuda") for _ in range(n_sets)]
    op = (C.c_void_p * n_sets)(*[t.data_ptr() for t in outs])
    stream = torch.cuda.current_stream().cuda_stream
    steps = max(200, args.steps)

    def run(mode, pol, n):
        ms = C.c_float(0.0)
        rc = P.pl_probe_store_shape(mode, pol, op, n_sets, n, C.c_void_p(stream), C.byref(ms))
        if rc != 0:
            raise RuntimeError("pl_probe_store_shape(%d, %d) failed with HIP error %d" % (mode, pol, rc))
        return ms.value * 1e3 / n

    settle(lambda: run(1, 0, 200))
    shapes = ["16 rows x 64 B", "4 rows x 256 B on sector boundaries", "8 rows x 128 B lines"]
    policies = ["sc1 nt", "nt", "plain"]
    rows = {}
    for rep_i in range(3):
        for m, shape in enumerate(shapes):
            for pol, pname in enumerate(policies):
                run(m, pol, 100)
                key = "%s, %s" % (shape, pname)
                rows[key] = round(min(run(m, pol, steps), rows.get(key, 1e9)), 2)
    # every pattern writes every float of a workgroup's rows exactly once
    for m in range(3):
        outs[0].fill_(float("nan"))
        run(m, 2, 1)
        torch.cuda.synchronize()
        assert not bool(torch.isnan(outs[0]).any()), "store pattern %d leaves floats unwritten" % m
    print(json.dumps({
        "metric": "store-only kernels over the metric shape's fp32 output: us per launch",
        "unit": "us", "n_gpus": 1, "steps": steps, "data": "synthetic",
        "config": {"workload": "store_shapes_c3_output", "output_MB": out_bytes / 1e6, "buffer_sets": n_sets, "grid": "256 workgroups x 512 threads"},
        "us_per_launch": rows,
        "TBs": {k: round(out_bytes / (v * 1e-6) / 1e12, 2) for k, v in rows.items()},
    }))
    return 0


def run_floors(args):
    """What the device needs for the launch and the memory traffic of the
    metric shape (64 x 512 -> 512 @14x14, int8 -> fp32) without the
    arithmetic: the probes of bench_probes/floor_probes.hip on the
    image kernel's grid and rotating buffers, next to the image kernel itself.
    Not the headline metric: printed as its own JSON line."""
    import torch

    import helpers

    capi, wl = helpers.capi, helpers.workloads
    P = load_probes()
    P.pl_probe_floor.restype = C.c_int
    P.pl_probe_floor.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_float)]
    case = wl.CONFIGS["c3"]()
    kernel, weights = helpers.make_kernel(case, algo=capi.ALGO_AUTO)
    batch, ic, oc, hw = case.batch, case.dense.shape[1], case.dense.shape[0], case.im_size
    set_bytes = case.x.nbytes + batch * oc * hw * 4
    n_sets = int(LLC_BYTES * 1.25 // set_bytes) + 1
    x0 = torch.from_numpy(case.x).cuda()
    xs = [x0] + [x0.clone() for _ in range(n_sets - 1)]
    outs = [torch.empty((batch, oc) + tuple(case.x.shape[2:]), dtype=torch.float32, device="cuda") for _ in range(n_sets)]
    xp = (C.c_void_p * n_sets)(*[t.data_ptr() for t in xs])
    op = (C.c_void_p * n_sets)(*[t.data_ptr() for t in outs])
    stream = torch.cuda.current_stream().cuda_stream
    L = capi.lib()
    steps = max(200, args.steps)

    def probe(kind, n):
        ms = C.c_float(0.0)
        rc = P.pl_probe_floor(kind, xp, op, n_sets, batch, ic, oc, hw, n, C.c_void_p(stream), C.byref(ms))
        if rc != 0:
            raise RuntimeError("pl_probe_floor(%d) failed with HIP error %d" % (kind, rc))
        return ms.value * 1e3 / n

    def image(n):
        ms = C.c_float(0.0)
        capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, n_sets, batch, hw, n, C.c_void_p(stream), C.byref(ms)))
        return ms.value * 1e3 / n

    settle(lambda: image(200))
    names = ["empty", "write", "stream", "load", "load_write", "load_transpose_write", "load_transposing_reads_write"]
    rows = {}
    for rep_i in range(3):  # three rounds, the best of each
        for k, name in enumerate(names):
            probe(k, 100)
            us = probe(k, steps)
            rows[name] = round(min(us, rows.get(name, 1e9)), 2)
        image(100)
        rows["image_mfma_kernel"] = round(min(image(steps), rows.get("image_mfma_kernel", 1e9)), 2)
    nbytes = case.algorithmic_bytes(weights)
    print(json.dumps({
        "metric": "launch and memory floors of the metric shape: us per launch",
        "unit": "us", "n_gpus": 1, "steps": steps, "data": "synthetic",
        "config": {"workload": "floors_c3_shape", "shape": "N=%d %d->%d @%dx%d" % (batch, ic, oc, case.x.shape[2], case.x.shape[3]), "buffer_sets": n_sets, "grid": "%d workgroups x 512 threads (stream: 2048 x 256)" % (batch * oc // 128),
                   "input_MB": case.x.nbytes / 1e6, "output_MB": batch * oc * hw * 4 / 1e6},
        "us_per_launch": rows,
        "frac_of_8TBs_if_the_kernel_ran_at": {k: round(nbytes / (v * 1e-6) / 1e9 / HBM_PEAK_GBS, 3) for k, v in rows.items() if k != "empty" and k != "load"},
    }))
    return 0


def run_c5(args):
    """MobileNetV1-1.0 pointwise stack (13 layers, batch 64, int8 -> int8, 90 %
    unstructured zeros, relu) timed as one sequence of 13 launches per step.
    Layer i+1 consumes layer i's int8 output where the shapes chain (2->3,
    4->5, 6->7..11, 12->13); at the four spatial breaks (stride-2 depthwise
    layers of the real network, not part of this path) a fresh random tensor
    is fed.  Not the headline metric: printed as its own JSON line."""
    import numpy as np
    import torch

    import helpers

    capi, wl = helpers.capi, helpers.workloads
    L = capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    layers = []
    prev_out = None
    total_ops = total_bytes = 0.0
    for i in range(13):
        case = wl.config5_layer(i)
        if args.algo == "image":
            raise SystemExit("--algo image applies to single layers; the stack holds shapes outside the image kernel's range (use auto)")
        kernel, weights = helpers.make_kernel(case, algo={"auto": capi.ALGO_AUTO, "walk": capi.ALGO_ROW_WALK, "mfma": capi.ALGO_BLOCK_MFMA}[args.algo])
        ic, oc, hw = wl.MOBILENET_V1_POINTWISE[i]
        chained = prev_out is not None and tuple(prev_out.shape[1:]) == (ic, hw, hw)
        x = prev_out if chained else torch.from_numpy(case.x).cuda()
        out = torch.empty((case.batch, oc, hw, hw), dtype=torch.int8, device="cuda")
        # parity of this layer on its actual input (first two images)
        capi.check(L.pl_sparse_conv_run(kernel._handle, x.data_ptr(), out.data_ptr(), case.batch, hw * hw, C.c_void_p(stream)))
        torch.cuda.synchronize()
        want = helpers.run_oracle(case, x=x[:2].cpu().numpy())
        assert np.array_equal(out[:2].cpu().numpy(), want), "layer %d differs from the oracle" % (i + 1)
        layers.append((case, kernel, x, out))
        prev_out = out
        total_ops += case.algorithmic_ops()
        total_bytes += case.algorithmic_bytes(weights)

    def sequence(on_stream=None):
        st = stream if on_stream is None else on_stream
        for case, kernel, x, out in layers:
            capi.check(L.pl_sparse_conv_run(kernel._handle, x.data_ptr(), out.data_ptr(), case.batch, case.im_size, C.c_void_p(st)))

    settle(sequence)
    # per-layer kernel time (events around repeated launches of one layer)
    per_layer = []
    for case, kernel, x, out in layers:
        xp = (C.c_void_p * 1)(x.data_ptr())
        op = (C.c_void_p * 1)(out.data_ptr())
        ms = C.c_float(0.0)
        capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, 1, case.batch, case.im_size, 20, C.c_void_p(stream), None))
        capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, 1, case.batch, case.im_size, 100, C.c_void_p(stream), C.byref(ms)))
        per_layer.append(ms.value * 10.0)  # us per launch
    for _ in range(max(1, args.warmup // 13)):
        sequence()
    torch.cuda.synchronize()
    steps = max(1, args.steps // 13)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        sequence()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    seq_us = e0.elapsed_time(e1) * 1e3 / steps
    # the same 13 launches captured once as a HIP graph (kernel nodes only)
    # and replayed; every replay is compared with the eager results
    eager_last = [layers[i][3].clone() for i in (0, 6, 12)]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sequence(torch.cuda.current_stream().cuda_stream)
    graph_ok = True
    for _ in range(3):
        for i in (0, 6, 12):
            layers[i][3].zero_()
        graph.replay()
        torch.cuda.synchronize()
        graph_ok = graph_ok and all(torch.equal(layers[i][3], ref) for i, ref in zip((0, 6, 12), eager_last))
    g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    g0.record()
    for _ in range(steps):
        graph.replay()
    g1.record()
    torch.cuda.synchronize()
    graph_us = g0.elapsed_time(g1) * 1e3 / steps
    line = {
        "metric": "MobileNetV1 pointwise stack, int8, 90% sparse: nnz-GOP/s of the 13-launch sequence",
        "value": total_ops * steps / wall / 1e9,
        "unit": "nnz-GOP/s",
        "n_gpus": 1,
        "steps": steps,
        "ms_per_step": wall * 1e3 / steps,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "c5_mobilenet_v1_pointwise_stack", "batch": 64, "layers": 13},
        "roofline": {"bound": "hbm", "achieved": total_bytes / (seq_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": total_bytes / (seq_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "algorithmic_bytes_per_sequence": total_bytes, "sequence_us": seq_us, "sum_of_layer_kernel_us": sum(per_layer),
                     "graph_replay_us": graph_us, "graph_replay_matches_eager": graph_ok},
        "per_layer_kernel_us": [round(v, 2) for v in per_layer],
        "per_layer_frac": [round(c.algorithmic_bytes(helpers.pla.detect_and_pack(c.dense, c.im_size)) / (t * 1e-6) / 1e9 / HBM_PEAK_GBS, 3) for (c, _, _, _), t in zip(layers, per_layer)],
    }
    print(json.dumps(line))
    return 0


SMALL_BATCH_SHAPES = [(32, 64, 112), (64, 128, 56), (128, 128, 56), (128, 256, 28), (256, 256, 28), (256, 512, 14), (512, 512, 14), (512, 1024, 7), (1024, 1024, 7)]
SMALL_BATCHES = (1, 4, 16, 64)


def run_small_batch(args):
    """The nine distinct pointwise shapes of MobileNetV1-1.0 (int8 -> int8, relu, 90 % zeros) at 1, 4, 16 and
    64 images per launch: the algorithm a PL_ALGO_AUTO handle picks and its time next to every algorithm forced
    (helpers.algo_times: every handle parity-checked against the oracle, buffer sets rotated, the best of three
    timed runs).  One JSON line; `auto_over_best` is what the selection rule costs where it picks wrong."""
    import helpers

    wl = helpers.workloads
    rows = []
    worst = 0.0
    for ic, oc, hw in SMALL_BATCH_SHAPES:
        for batch in SMALL_BATCHES:
            case = wl.config5_layer(wl.MOBILENET_V1_POINTWISE.index((ic, oc, hw)), batch=batch)
            times, picked = helpers.algo_times(case, warm=100, steps=500)
            best = min(v for k, v in times.items() if k != "auto")
            worst = max(worst, times["auto"] / best)
            rows.append({"shape": "%d->%d @%dx%d" % (ic, oc, hw, hw), "batch": batch, "auto_picks": picked, "us": {k: round(v, 2) for k, v in times.items()}, "auto_over_best": round(times["auto"] / best, 3),
                         "frac_of_8TBs": round(case.algorithmic_bytes(helpers.pla.detect_and_pack(case.dense, case.im_size)) / (times["auto"] * 1e-6) / 1e9 / HBM_PEAK_GBS, 3)})
    print(json.dumps({"metric": "int8 pointwise layers of MobileNetV1 at small batch: us per launch by algorithm", "unit": "us", "n_gpus": 1, "data": "synthetic", "dtype": "int8",
                      "config": {"workload": "small_batch_int8", "sparsity": 0.9, "parity_checked": True}, "worst_auto_over_best": round(worst, 3), "rows": rows}))
    return 0


def run_lite_program_bench(batch):
    """The same body through the C++ operator surface (op descriptions -> detect pass -> chain pass ->
    mir::HipProgram), measured by bench_probes/lite_program_bench in a process of its own: host time per
    step, the eager sequence and its replay as a HIP graph.  None when the program is not built."""
    import subprocess

    exe = os.path.join(ROOT, "bench_probes", "lite_program_bench")
    if not os.path.exists(exe):
        return None
    res = subprocess.run([exe, "--batch", str(batch), "--sequences", "40"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    if res.returncode != 0:
        raise RuntimeError("lite_program_bench failed (%d): %s" % (res.returncode, res.stderr[-2000:]))
    return json.loads(res.stdout.strip().splitlines()[-1])


def run_mobilenet(args):
    """The convolutional body of MobileNetV1-1.0 at batch 64 in int8: thirteen
    times (depthwise 3x3, relu) then (pointwise 1x1 through sparse_conv2d, 90 %
    zeros, relu), every layer consuming the previous layer's int8 output: 26
    launches per step.  Every layer is compared with the oracle on the first
    two images of its actual input.  Not the headline metric: printed as its
    own JSON line."""
    import numpy as np
    import torch

    import helpers
    from oracle import oracle as O

    capi, wl, pla = helpers.capi, helpers.workloads, helpers.pla
    L = capi.lib()
    stream = torch.cuda.current_stream().cuda_stream
    batch = 64
    rng = np.random.RandomState(5)
    x = torch.from_numpy(rng.randint(-127, 128, size=(batch, 32, 112, 112)).astype(np.int8)).cuda()
    keep_input = x  # the launches below hold device addresses, not tensors: the tensors must stay alive
    steps_list = []  # (kind, name, launch, bytes)
    keep = []
    total_bytes = 0.0
    nonzero = []
    for i in range(13):
        dwc = wl.config5_depthwise_layer(i)
        param = pla.ConvParam(dwc.filter, dwc.bias, strides=(dwc.stride, dwc.stride), paddings=(1, 1, 1, 1), activation_param=dwc.act, input_scale=dwc.input_scale,
                              weight_scale=dwc.weight_scale, output_scale=dwc.output_scale)
        dw = pla.DepthwiseConv(param, out_precision="int8")
        dw.PrepareForRun()
        t = dw.Run(x)
        torch.cuda.synchronize()
        a = O.Act()
        a.type = 1
        want = O.dwconv3x3_int8(x[:2].cpu().numpy(), dwc.filter[:, 0], dw.w_scale_, dw.bias_, a, out="int8", stride=dwc.stride, pad=1)
        assert np.array_equal(t[:2].cpu().numpy(), want), "depthwise layer %d differs from the oracle" % (i + 1)
        dw_bytes = dwc.algorithmic_bytes(batch)
        # the C entry point itself: the kernel class's argument checks cost more host time per launch than the small layers run
        steps_list.append(("depthwise", dwc.name, (lambda h=dw._handle, xp=C.c_void_p(x.data_ptr()), tp=C.c_void_p(t.data_ptr()), size=dwc.in_size: capi.check(
            L.pl_dwconv3x3_run(h, xp, tp, batch, size, size, C.c_void_p(stream)))), dw_bytes))
        case = wl.config5_layer(i)
        kernel, weights = helpers.make_kernel(case)
        ic, oc, hw = wl.MOBILENET_V1_POINTWISE[i]
        out = torch.empty((batch, oc, hw, hw), dtype=torch.int8, device="cuda")
        capi.check(L.pl_sparse_conv_run(kernel._handle, t.data_ptr(), out.data_ptr(), batch, hw * hw, C.c_void_p(stream)))
        torch.cuda.synchronize()
        assert np.array_equal(out[:2].cpu().numpy(), helpers.run_oracle(case, x=t[:2].cpu().numpy())), "pointwise layer %d differs from the oracle" % (i + 1)
        pw_bytes = case.algorithmic_bytes(weights)
        steps_list.append(("pointwise", case.name, (lambda h=kernel._handle, ti=t, oi=out, n=hw * hw: capi.check(L.pl_sparse_conv_run(h, ti.data_ptr(), oi.data_ptr(), batch, n, C.c_void_p(stream)))), pw_bytes))
        keep.append((dw, kernel, t, out))
        nonzero.append(round(float((out != 0).float().mean().item()), 3))
        total_bytes += dw_bytes + pw_bytes
        x = out

    def sequence():
        for _, _, launch, _ in steps_list:
            launch()

    # The same body with every pointwise layer that can do so running the depthwise layer behind it in its own
    # launch (pl_sparse_conv_dwconv3x3_run: 14 x 14 maps; the tensor between the two is not written).
    fused_list, fused_pairs = [], []
    i = 0
    while i < len(steps_list):
        if steps_list[i][0] == "pointwise" and i + 1 < len(steps_list):
            li = i // 2  # pointwise layer li, followed by the depthwise layer in front of pointwise layer li + 1
            kernel, (dw_next, _, t_next, _) = keep[li][1], keep[li + 1]
            size = wl.MOBILENET_V1_POINTWISE[li][2]
            if L.pl_sparse_conv_dwconv3x3_pays(kernel._handle, dw_next._handle, batch, size, size):
                t_in = keep[li][2]
                fused_list.append(lambda hc=kernel._handle, hd=dw_next._handle, xi=t_in, oi=t_next, n=size: capi.check(
                    L.pl_sparse_conv_dwconv3x3_run(hc, hd, C.c_void_p(xi.data_ptr()), C.c_void_p(oi.data_ptr()), batch, n, n, C.c_void_p(stream))))
                fused_pairs.append("%s + %s" % (steps_list[i][1], steps_list[i + 1][1]))
                i += 2
                continue
        fused_list.append(steps_list[i][2])
        i += 1

    def fused_sequence():
        for launch in fused_list:
            launch()

    sequence()
    torch.cuda.synchronize()
    final_two_launches = keep[-1][3].clone()
    keep[-1][3].zero_()
    fused_sequence()
    torch.cuda.synchronize()
    fused_equal = bool(torch.equal(final_two_launches, keep[-1][3]))

    settle(sequence)
    per_layer = []
    for kind, name, launch, nbytes in steps_list:
        for _ in range(10):
            launch()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(50):
            launch()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / 50
        per_layer.append({"layer": name, "kind": kind, "kernel_us": round(us, 2), "frac": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 3)})
    for _ in range(max(1, args.warmup // 26)):
        sequence()
    torch.cuda.synchronize()
    steps = max(1, args.steps // 26)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        sequence()
    e1.record()
    host_us = (time.perf_counter() - t0) * 1e6 / steps  # time the host needs to enqueue one sequence
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    seq_us = e0.elapsed_time(e1) * 1e3 / steps
    for _ in range(max(1, args.warmup // 26)):
        fused_sequence()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(steps):
        fused_sequence()
    e1.record()
    torch.cuda.synchronize()
    fused_seq_us = e0.elapsed_time(e1) * 1e3 / steps
    dw_us = sum(p["kernel_us"] for p in per_layer if p["kind"] == "depthwise")
    pw_us = sum(p["kernel_us"] for p in per_layer if p["kind"] == "pointwise")
    print(json.dumps({
        "lite_program": None if args.no_lite_program else run_lite_program_bench(batch),
        "lite_program_batch_1": None if args.no_lite_program else run_lite_program_bench(1),
        "metric": "MobileNetV1-1.0 convolutional body, int8, batch 64: images/s of the 26-launch sequence",
        "value": batch * steps / wall,
        "unit": "images/s",
        "n_gpus": 1,
        "steps": steps,
        "ms_per_step": wall * 1e3 / steps,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "mobilenet_v1_body_int8", "batch": batch, "launches": 26, "pointwise_sparsity": 0.9, "parity_checked": True},
        "roofline": {"bound": "hbm", "achieved": total_bytes / (seq_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": total_bytes / (seq_us * 1e-6) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "algorithmic_bytes_per_sequence": total_bytes, "sequence_us": seq_us, "host_enqueue_us_per_sequence": round(host_us, 1), "sum_depthwise_kernel_us": round(dw_us, 1), "sum_pointwise_kernel_us": round(pw_us, 1)},
        "pairs_in_one_launch": {"pairs": fused_pairs, "launches": len(fused_list), "sequence_us": fused_seq_us, "output_equals_two_launches": fused_equal},
        "per_layer": per_layer,
        "nonzero_fraction_of_pointwise_outputs": nonzero,
    }))
    return 0


def main():
    args = parse()
    if args.gpus != 1:
        sys.stderr.write("bench.py measures one GPU; --gpus %d is not supported: this path shards over images with no exchange between GPUs, so N GPUs would each run this same kernel on their share of the batch\n" % args.gpus)
        return 2
    import numpy as np
    import torch

    import helpers

    capi, wl = helpers.capi, helpers.workloads
    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs a GPU\n")
        return 2
    torch.cuda.set_device(0)
    if args.config == "density-sweep":
        return run_density_sweep(args)
    if args.config == "floors":
        return run_floors(args)
    if args.config == "store-shapes":
        return run_store_shapes(args)
    if args.config == "device-rates":
        return run_device_rates(args)
    if args.config == "c5":
        return run_c5(args)
    if args.config == "calib":
        return run_calib(args)
    if args.config == "mobilenet":
        return run_mobilenet(args)
    if args.config == "small-batch":
        return run_small_batch(args)
    if args.config == "float-layers":
        return run_float_layers(args)
    if args.config == "custom":
        case = custom_case(args)
        args.fp16 = args.fp16 or args.kind == "fp16"
    else:
        case = wl.CONFIGS[args.config]()
    if args.fp16:
        if case.kind != capi.KIND_FP32:
            sys.stderr.write("--fp16 applies to the fp32 configurations\n")
            return 2
        case.kind = capi.KIND_FP16
        case.x = case.x.astype(np.float16)
        case.name += "_fp16"
        args.no_cpu_baseline = True  # the CPU baselines are fp32 / int8 paths
    algo = {"auto": capi.ALGO_AUTO, "walk": capi.ALGO_ROW_WALK, "mfma": capi.ALGO_BLOCK_MFMA, "image": capi.ALGO_IMAGE_MFMA}[args.algo]
    tune = capi.tuning(image_kernel={"rule": 0, "regroup": capi.IMAGE_KERNEL_REGROUP, "transpose": capi.IMAGE_KERNEL_TRANSPOSE, "rows": capi.IMAGE_KERNEL_ROWS}[args.image_kernel],
                       image_tr_regroup=capi.TUNE_NEVER if args.image_regroup == "valu" else capi.TUNE_RULE)
    kernel, weights = helpers.make_kernel(case, algo=algo, tuning=tune)
    info = kernel.info()
    ops = case.algorithmic_ops()
    nbytes = case.algorithmic_bytes(weights)

    # rotating buffer sets: footprint above the last-level cache
    out_dtype = {capi.KIND_FP32: torch.float32, capi.KIND_INT8_FP32: torch.float32, capi.KIND_INT8_INT8: torch.int8, capi.KIND_FP16: torch.float16}[case.kind]
    oc = case.dense.shape[0]
    set_bytes = case.x.nbytes + case.batch * oc * case.im_size * {torch.int8: 1, torch.float16: 2}.get(out_dtype, 4)
    n_sets = 1 if args.cache_resident else int(LLC_BYTES * 1.25 // set_bytes) + 1
    x0 = torch.from_numpy(case.x).cuda()
    xs = [x0] + [x0.clone() for _ in range(n_sets - 1)]
    outs = [torch.empty((case.batch, oc) + tuple(case.x.shape[2:]), dtype=out_dtype, device="cuda") for _ in range(n_sets)]
    xp = (C.c_void_p * n_sets)(*[t.data_ptr() for t in xs])
    op = (C.c_void_p * n_sets)(*[t.data_ptr() for t in outs])
    stream = torch.cuda.current_stream().cuda_stream
    L = capi.lib()

    def sequence(steps, timed):
        ms = C.c_float(0.0)
        capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp, op, n_sets, case.batch, case.im_size, steps, C.c_void_p(stream), C.byref(ms) if timed else None))
        return ms.value

    # parity of what is being timed (first set) against the oracle on a slice
    sequence(min(n_sets, 2), False)
    torch.cuda.synchronize()
    nchk = min(case.batch, 2)
    want = helpers.run_oracle(case, x=case.x[:nchk])
    got = outs[0][:nchk].cpu().numpy()
    if case.kind == capi.KIND_FP16:
        assert np.array_equal(got, want), "timed kernel output differs from the oracle"
    elif case.kind == capi.KIND_FP32:
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    else:
        assert np.array_equal(got, want), "timed kernel output differs from the oracle"

    settle(lambda: sequence(200, False))
    sequence(args.warmup, False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev_ms = sequence(args.steps, True)  # events on the launch stream bracket exactly the timed steps
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    ms_per_step = wall * 1e3 / args.steps
    kernel_ms = ev_ms / args.steps

    # labelled extras: the same kernel on one buffer set (inputs and outputs
    # stay in the last-level cache), and what a plain device copy reaches on
    # this box (1 GiB each way per launch)
    xp1 = (C.c_void_p * 1)(xs[0].data_ptr())
    op1 = (C.c_void_p * 1)(outs[0].data_ptr())
    ms1 = C.c_float(0.0)
    capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp1, op1, 1, case.batch, case.im_size, 50, C.c_void_p(stream), None))
    capi.check(L.pl_sparse_conv_run_sequence(kernel._handle, xp1, op1, 1, case.batch, case.im_size, 200, C.c_void_p(stream), C.byref(ms1)))
    cache_resident_us = ms1.value * 1e3 / 200
    copy_gbs = None
    if not args.copy_calibration:  # counter runs keep the 64 MiB calibration copy as their only large copy
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        c0.record()
        for _ in range(10):
            dst.copy_(src)
        c1.record()
        torch.cuda.synchronize()
        copy_gbs = 2.0 * (1 << 30) * 10 / (c0.elapsed_time(c1) * 1e-3) / 1e9
        del src, dst
    achieved = nbytes / (kernel_ms * 1e-3) / 1e9
    algo_names = {capi.ALGO_ROW_WALK: "row_walk", capi.ALGO_BLOCK_MFMA: "block_mfma", capi.ALGO_IMAGE_MFMA: "image_mfma"}
    algo_name = algo_names[capi.check(L.pl_sparse_conv_algo_for(kernel._handle, case.batch, case.im_size))]
    traffic, traffic_detail = measured_traffic(case.name, algo_name)
    # int8: the same launch through every algorithm the shape allows (same rotating buffers, 200 untimed then 1000 timed launches each)
    per_algo = None
    if case.kind in (capi.KIND_INT8_FP32, capi.KIND_INT8_INT8):
        per_algo = {algo_name: round(kernel_ms * 1e3, 3)}
        others = sorted(algo_names.items())
        if algo_name == "image_mfma":
            others.append((capi.ALGO_IMAGE_MFMA, "image_mfma_regroup_in_lds"))  # a pair of wavefronts per two row tiles, image landed in LDS and regrouped there
            others.append((capi.ALGO_IMAGE_MFMA, "image_mfma_valu_regroup"))  # the same with the regrouping done by the vector ALU
            others.append((capi.ALGO_IMAGE_MFMA, "image_mfma_transposing_reads"))  # the image kernel that never regroups
        for a, name in others:
            if name in per_algo:
                continue
            try:
                other_tune = {"image_mfma_regroup_in_lds": capi.tuning(image_kernel=capi.IMAGE_KERNEL_REGROUP),
                              "image_mfma_valu_regroup": capi.tuning(image_kernel=capi.IMAGE_KERNEL_REGROUP, image_tr_regroup=capi.TUNE_NEVER),
                              "image_mfma_transposing_reads": capi.tuning(image_kernel=capi.IMAGE_KERNEL_TRANSPOSE)}.get(name)
                other, _ = helpers.make_kernel(case, algo=a, tuning=other_tune)
            except capi.SparseConvError:
                continue  # this shape is outside the algorithm's range
            if L.pl_sparse_conv_run_sequence(other._handle, xp, op, n_sets, case.batch, case.im_size, 200, C.c_void_p(stream), None) < 0:
                continue
            torch.cuda.synchronize()
            assert np.array_equal(outs[0][:nchk].cpu().numpy(), want), "%s output differs from the oracle" % name
            ms_o = C.c_float(0.0)
            capi.check(L.pl_sparse_conv_run_sequence(other._handle, xp, op, n_sets, case.batch, case.im_size, 1000, C.c_void_p(stream), C.byref(ms_o)))
            per_algo[name] = round(ms_o.value * 1e3 / 1000, 3)
    line = {
        "metric": METRICS[args.config] + (" (half-precision kernel)" if args.fp16 else ""),
        "value": ops * args.steps / wall / 1e9,
        "unit": "nnz-GOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {capi.KIND_FP32: "f32", capi.KIND_FP16: "f16"}.get(case.kind, "int8"),
        "data": "synthetic",
        "config": {
            "workload": case.name,
            "shape": "N=%d %d->%d @%dx%d" % (case.batch, case.dense.shape[1], oc, case.x.shape[2], case.x.shape[3]),
            "nnz": case.nnz,
            "sparsity": 1.0 - case.nnz / float(case.dense.size),
            "flag_semi": weights.flag_semi,
            "algo": algo_name,
            "weight_blocks_present": [info["mfma_blocks"], info["mfma_blocks_total"]],
            "buffer_sets": n_sets,
            "rotation_MB": n_sets * set_bytes / 1e6,
            "parity_checked": True,
            "clock_settle_ms": SETTLE_S * 1e3,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_source": "profiles/hbm_traffic.json (separate rocprofv3 --pmc runs)" if traffic else None,
            "traffic_detail": traffic_detail,
            "algorithmic_bytes_per_launch": nbytes,
            "kernel_us": kernel_ms * 1e3,
            "nnz_TOPs_kernel": ops / (kernel_ms * 1e-3) / 1e12,
            "measured_copy_GBs": copy_gbs,
            "frac_of_measured_copy": achieved / copy_gbs if copy_gbs else None,
            "cache_resident_kernel_us": cache_resident_us,
            "kernel_us_by_algorithm": per_algo,
        },
    }
    if args.copy_calibration:
        src = torch.randint(0, 255, (COPY_CALIBRATION_BYTES,), dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        line["config"]["copy_calibration_bytes"] = COPY_CALIBRATION_BYTES
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(case, weights)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Shared plumbing of the parity tests: run one workload through the HIP
library (via the C ABI) and through the CPU oracle with identical merged
parameters."""
import importlib

import numpy as np

from oracle import oracle as O

pla = importlib.import_module("paddle-lite_amd")
capi = pla.capi
workloads = importlib.import_module("paddle-lite_amd.workloads")


def oracle_act(ap):
    """ActivationParam (already merged) -> oracle activation struct."""
    t = ap.active_type if ap.has_active else O.ACT_NONE
    return O.Act(t, ap.Relu_clipped_coef, ap.Leaky_relu_alpha, ap.hard_swish_scale, ap.hard_swish_offset, ap.hard_swish_threshold)


def merged_for_oracle(case, quirks=False):
    """Scale / bias / activation constants the math functions receive, derived
    here with explicit numpy float32 arithmetic (not through the package)."""
    act = case.act.copy()
    bias = case.bias
    if case.kind in (capi.KIND_FP32, capi.KIND_FP16):
        return None, bias, oracle_act(act)
    ws = np.asarray(case.weight_scale, np.float32)
    if ws.size == 1:
        ws = np.repeat(ws, case.dense.shape[0])
    isc, osc = np.float32(case.input_scale), np.float32(case.output_scale)
    if case.kind != capi.KIND_INT8_INT8:
        return (ws * isc).astype(np.float32), bias, oracle_act(act)
    scale = (ws * isc / osc).astype(np.float32)
    if bias is not None:
        bias = (bias / osc).astype(np.float32)
    d = lambda v: float(np.float32(np.float32(v) / osc))  # noqa: E731
    if act.active_type == O.ACT_RELU6:
        act.Relu_clipped_coef = d(act.Relu_clipped_coef)
    if act.active_type == O.ACT_LEAKY_RELU and quirks:
        act.Leaky_relu_alpha = d(act.Leaky_relu_alpha)
    if act.active_type == O.ACT_HARD_SWISH:
        act.hard_swish_scale = d(act.hard_swish_scale)
        act.hard_swish_offset = d(act.hard_swish_offset)
        act.hard_swish_threshold = d(act.hard_swish_threshold)
        if quirks:  # the math function divides these two once more
            act.hard_swish_offset = d(act.hard_swish_offset)
            act.hard_swish_threshold = d(act.hard_swish_threshold)
    return scale, bias, oracle_act(act)


def oracle_pack(case, force_semi=None):
    if force_semi is None:
        return O.pack_like_pass(case.dense, case.im_size)
    if force_semi:
        return O.pack(case.dense, case.im_size, O.LAYOUT_SEMI)
    return O.pack(case.dense, case.im_size, O.LAYOUT_PADDED if case.dense.dtype == np.float32 else O.LAYOUT_UNPADDED)


def run_oracle(case, packed=None, quirks=False, x=None):
    pk = packed or oracle_pack(case)
    x = case.x if x is None else x
    scale, bias, act = merged_for_oracle(case, quirks)
    if case.kind == capi.KIND_FP32:
        return O.sparse_conv_fp32(pk, x, bias, act)
    if case.kind == capi.KIND_FP16:
        return O.sparse_conv_fp16(pk, x, bias, act)
    if case.kind == capi.KIND_INT8_ACC32:
        return O.sparse_conv_int8_acc(pk, x)
    return O.sparse_conv_int8(pk, x, scale, bias, act, out_int8=(case.kind == capi.KIND_INT8_INT8))


_PREC = {capi.KIND_FP32: ("float32", "float32"), capi.KIND_INT8_FP32: ("int8", "float32"), capi.KIND_INT8_INT8: ("int8", "int8"), capi.KIND_INT8_ACC32: ("int8", "int32"), capi.KIND_FP16: ("float16", "float16")}


def make_kernel(case, algo=capi.ALGO_AUTO, force_semi=None, quirks=False, im_size=None, tuning=None):
    weights = pla.detect_and_pack(case.dense, im_size or case.im_size, force_semi=force_semi)
    param = pla.SparseConvParam(weights, bias=case.bias, activation_param=case.act, enable_int8=case.kind not in (capi.KIND_FP32, capi.KIND_FP16), input_scale=case.input_scale,
                                weight_scale=case.weight_scale if case.weight_scale is not None else (), output_scale=case.output_scale)
    prec = _PREC[case.kind]
    k = pla.SparseConvKernel(param, prec[0], prec[1], algo=algo, reference_quirks=quirks, tuning=tuning)
    k.PrepareForRun()
    return k, weights


def run_hip(case, algo=capi.ALGO_AUTO, force_semi=None, quirks=False, x=None, kernel=None, tuning=None):
    import torch

    k = kernel or make_kernel(case, algo, force_semi, quirks, tuning=tuning)[0]
    xd = torch.from_numpy(case.x if x is None else x).cuda()
    out = k.Run(xd)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def assert_same(case, got, want, what=""):
    assert got.shape == want.shape and got.dtype == want.dtype, (what, got.shape, want.shape, got.dtype, want.dtype)
    if case.kind == capi.KIND_FP16:
        # fp16: the same sequence of half-precision instructions -> the same
        # values (zeros compare equal whatever their sign)
        bad = ~((got == want) | (np.isnan(got) & np.isnan(want)))
        assert not bad.any(), "%s: %d of %d fp16 values differ, first %r vs %r" % (what, int(bad.sum()), got.size, got[bad][0], want[bad][0])
        return
    if case.kind == capi.KIND_FP32:
        # fp32: 1e-5 relative (the reference's own tests allow 1e-4 / 5e-5)
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6, err_msg=what)
    else:
        # int8 paths: exact integer accumulators and one fmaf -> bit-exact
        if not np.array_equal(got, want):
            bad = np.argwhere(got != want)
            raise AssertionError("%s: %d of %d elements differ, first at %s: got %r want %r" % (what, len(bad), got.size, tuple(bad[0]), got[tuple(bad[0])], want[tuple(bad[0])]))


ALGO_NAMES = {capi.ALGO_ROW_WALK: "row_walk", capi.ALGO_BLOCK_MFMA: "block_mfma", capi.ALGO_IMAGE_MFMA: "image_mfma"}


def algo_times(case, warm=100, steps=500, repeats=3, max_sets=24, rotation_bytes=320 << 20):
    """Device time per launch (us, events inside pl_sparse_conv_run_sequence) of an int8 case with the
    algorithm left to the handle ("auto") and with each algorithm forced; an algorithm the shape is outside of
    is left out.  Every handle's output on the first two images is compared with the oracle before it is
    timed.  Buffer sets rotate (up to `max_sets` of them, `rotation_bytes` in all); the runs of the handles are
    interleaved `repeats` times and the smallest time of each is kept, so that a clock ramp or another
    process's burst does not land on one algorithm.  Returns (times, name of the algorithm auto picked)."""
    import ctypes as C

    import torch

    L = capi.lib()
    oc = case.dense.shape[0]
    out_dtype = {capi.KIND_INT8_FP32: torch.float32, capi.KIND_INT8_INT8: torch.int8}[case.kind]
    set_bytes = case.x.nbytes + case.batch * oc * case.im_size * (1 if out_dtype == torch.int8 else 4)
    n_sets = max(1, min(max_sets, int(rotation_bytes // set_bytes) + 1))
    x0 = torch.from_numpy(case.x).cuda()
    xs = [x0] + [x0.clone() for _ in range(n_sets - 1)]
    outs = [torch.empty((case.batch, oc) + tuple(case.x.shape[2:]), dtype=out_dtype, device="cuda") for _ in range(n_sets)]
    xp = (C.c_void_p * n_sets)(*[t.data_ptr() for t in xs])
    op = (C.c_void_p * n_sets)(*[t.data_ptr() for t in outs])
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    nchk = min(case.batch, 2)
    want = run_oracle(case, x=case.x[:nchk])
    handles = {}
    for name, algo in [("auto", capi.ALGO_AUTO)] + [(n, a) for a, n in sorted(ALGO_NAMES.items())]:
        try:
            k, _ = make_kernel(case, algo=algo)
        except capi.SparseConvError:
            continue
        outs[0].zero_()
        if L.pl_sparse_conv_run_sequence(k._handle, xp, op, n_sets, case.batch, case.im_size, 1, stream, None) < 0:
            continue  # outside this algorithm's range at this batch or map size
        torch.cuda.synchronize()
        assert np.array_equal(outs[0][:nchk].cpu().numpy(), want), "%s: %s differs from the oracle" % (case.name, name)
        handles[name] = k
    picked = ALGO_NAMES[capi.check(L.pl_sparse_conv_algo_for(handles["auto"]._handle, case.batch, case.im_size))]
    times = {}
    for _ in range(repeats):
        for name, k in handles.items():
            capi.check(L.pl_sparse_conv_run_sequence(k._handle, xp, op, n_sets, case.batch, case.im_size, warm, stream, None))
            ms = C.c_float(0.0)
            capi.check(L.pl_sparse_conv_run_sequence(k._handle, xp, op, n_sets, case.batch, case.im_size, steps, stream, C.byref(ms)))
            us = ms.value * 1e3 / steps
            times[name] = min(times.get(name, us), us)
    return times, picked

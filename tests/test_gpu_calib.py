"""fp32 <-> int8 precision changes (the reference's calib op) on the GPU,
through the C ABI, against the oracle's restatement of fp32_to_int8 /
int8_to_fp32: bit-exact both ways."""
import importlib

import numpy as np
import pytest

from helpers import capi
from oracle import oracle as O

pytestmark = pytest.mark.gpu
pla = importlib.import_module("paddle-lite_amd")


def _run(cls, x_np, out_dtype, scale, offset_in=0, offset_out=0):
    import torch

    n = x_np.size
    xin = torch.zeros(n + 64, dtype=torch.from_numpy(x_np[:1].copy()).dtype, device="cuda")
    xin[offset_in:offset_in + n] = torch.from_numpy(x_np).cuda()
    out = torch.full((n + 64,), 77, dtype=out_dtype, device="cuda")
    k = cls(pla.CalibParam(xin[offset_in:offset_in + n], out[offset_out:offset_out + n], scale))
    k.PrepareForRun()
    k.Run(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    host = out.cpu().numpy()
    # nothing outside the destination range is touched
    assert (host[:offset_out] == 77).all() and (host[offset_out + n:] == 77).all()
    return host[offset_out:offset_out + n]


@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 255, 4096, 100003, 1 << 20])
@pytest.mark.parametrize("offsets", [(0, 0), (1, 3), (3, 13), (2, 16)])
def test_fp32_to_int8_bit_exact(n, offsets):
    import torch

    rng = np.random.RandomState(n % 977 + offsets[0])
    scale = 0.0371
    x = (rng.standard_normal(n) * 2.5).astype(np.float32)
    if n >= 16:
        # ties, the value just below one half, saturation both ways, zeros
        x[:12] = np.array([0.5, -0.5, 1.5, -2.5, 0.49999997, -0.49999997, 126.5, 127.4, 500.0, -500.0, 0.0, -0.0], dtype=np.float32) * np.float32(scale)
    got = _run(pla.CalibComputeFp32ToInt8, x, torch.int8, scale, *offsets)
    want = O.fp32_to_int8(x, scale)
    assert np.array_equal(got, want)
    if n:
        assert got.min() >= -127


@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 255, 4096, 100003, 1 << 20])
@pytest.mark.parametrize("offsets", [(0, 0), (1, 3), (3, 13), (16, 2)])
def test_int8_to_fp32_bit_exact(n, offsets):
    import torch

    rng = np.random.RandomState(n % 971 + offsets[1])
    x = rng.randint(-128, 128, size=n).astype(np.int8)
    got = _run(pla.CalibComputeInt8ToFp32, x, torch.float32, 0.0123, *offsets)
    want = O.int8_to_fp32(x, 0.0123)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_round_trip_of_representable_values():
    import torch

    scale = 0.25  # power of two: q * scale and its inverse are exact
    q = np.arange(-127, 128, dtype=np.int8).repeat(37)
    f = _run(pla.CalibComputeInt8ToFp32, q, torch.float32, scale)
    back = _run(pla.CalibComputeFp32ToInt8, f, torch.int8, scale)
    assert np.array_equal(back, q)


def test_bad_arguments_are_refused():
    L = capi.lib()
    assert L.pl_calib_fp32_to_int8(None, None, 16, 1.0, None) == capi.PL_ERR_BAD_ARG
    assert L.pl_calib_fp32_to_int8(None, None, -1, 1.0, None) == capi.PL_ERR_BAD_ARG
    assert L.pl_calib_int8_to_fp32(None, None, 0, 0.0, None) == capi.PL_ERR_BAD_ARG
    assert L.pl_calib_int8_to_fp32(None, None, 0, 1.0, None) == capi.PL_OK

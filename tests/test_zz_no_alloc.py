"""The sampler's entry point that allocates nothing (``lyp_sample_static``),
called through ctypes as a caller outside this package would, against the
entry point it is a variant of (``lyp_sample`` with a workspace from the
caller): two calls in a row on the same GPU, the second with fewer and shorter
rows, so that what the first call left in the built-in array is still there
when the second one runs."""
import ctypes
from ctypes import c_int, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def lib():
    from lyapunov_engine_amd.kernels import build, ops

    ops.require_gpu()
    lib = ctypes.CDLL(str(build.core_library()))
    lib.lyp_last_error.restype = ctypes.c_char_p
    lib.lyp_sample_static.argtypes = [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_void_p]
    lib.lyp_sample_static.restype = c_int
    lib.lyp_sample_static_max_rows.restype = c_int
    return lib


def _inputs(rows, V, seed):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(rows, V, generator=g) * 3
    temperature = torch.tensor([0.0, 0.8, 1.3, 0.0, 0.7, 1.0, 0.9, 0.0, 1.1][:rows])
    top_k = torch.tensor([-1, -1, 40, -1, -1, 5, 100, -1, 17][:rows], dtype=torch.int32)
    top_p = torch.tensor([1.0, 1.0, 1.0, 1.0, 0.6, 0.9, 0.95, 1.0, 0.8][:rows])
    uniform = torch.rand(rows, generator=g)
    return [t.to(DEV) for t in (logits, temperature, top_k, top_p, uniform)]


def _static(lib, logits, temperature, top_k, top_p, uniform):
    rows, V = logits.shape
    out = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    rc = lib.lyp_sample_static(logits.data_ptr(), logits.stride(0), rows, V, temperature.data_ptr(), top_k.data_ptr(),
                               top_p.data_ptr(), uniform.data_ptr(), out.data_ptr(), None,
                               torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.lyp_last_error().decode()
    torch.cuda.synchronize()
    return out.cpu(), free_before - torch.cuda.mem_get_info()[0]


def _with_workspace(logits, temperature, top_k, top_p, uniform):
    from lyapunov_engine_amd.kernels import ops

    rows = logits.shape[0]
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops.sample(logits, temperature, top_k, top_p, uniform, out, ops.sample_workspace(rows, DEV))
    return out.cpu()


def test_static_sampler_equals_the_one_with_a_workspace(lib):
    first = _inputs(9, 1003, seed=11)
    second = _inputs(3, 515, seed=12)          # fewer rows, a shorter vocabulary
    got1, _ = _static(lib, *first)             # the first call on the device also looks the array's address up
    got2, taken = _static(lib, *second)
    assert got1.tolist() == _with_workspace(*first).tolist()
    assert got2.tolist() == _with_workspace(*second).tolist()
    assert int(first[0][0].argmax()) == got1[0] and int(second[0][0].argmax()) == got2[0]   # greedy rows
    assert taken == 0, f"the device's free memory shrank by {taken} bytes over a call"


def test_static_sampler_refuses_more_rows_than_its_array_holds(lib):
    most = lib.lyp_sample_static_max_rows()
    assert most >= 64
    rc = lib.lyp_sample_static(None, 8, most + 1, 8, None, None, None, None, None, None, None)
    assert rc != 0 and str(most) in lib.lyp_last_error().decode()

"""Code objects loaded at run time (ahip_module_load / ahip_launch): the sample module built from
altius_amd/csrc/modules/scale_shift.hip is launched by kernel name on the context's stream and
checked against the oracle; bad images, unknown names and impossible launch shapes are refused on
the host before anything reaches the device."""
import ctypes
import os

import numpy as np
import pytest

from altius_amd import _lib
from altius_amd import build as B
from altius_amd import device as D
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def image():
    path = B.module_path("scale_shift")
    assert os.path.exists(path), "altius_amd/modules/scale_shift.hsaco is not built (python -m altius_amd.build)"
    with open(path, "rb") as f:
        return f.read()


@pytest.fixture()
def module(ctx, image):
    m = ctx.load_module(image)
    yield m
    ctx.unload_module(m)


def test_module_hard_sigmoid_matches_oracle(ctx, oracle, case, module):
    case("module kernel ahip_module_hard_sigmoid, n=100003")
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(100003) * 4).astype(np.float32)
    x[:4] = [np.nan, np.inf, -np.inf, -0.0]
    alpha, beta = np.float32(1.0 / 6.0), np.float32(0.5)
    din, dout = ctx.upload(x), ctx.alloc(x.nbytes)
    n = x.size
    ctx.launch(module, "ahip_module_hard_sigmoid", ((n + 255) // 256, 1, 1), (256, 1, 1),
               [ctypes.c_void_p(dout.ptr), ctypes.c_void_p(din.ptr), ctypes.c_float(alpha), ctypes.c_float(beta),
                ctypes.c_uint64(n)])
    got = ctx.download(dout, x.shape)
    assert_bits_equal(got, oracle.unary(oracle.HARDSIGMOID, x, alpha=float(alpha), beta=float(beta)), "module hardsigmoid")
    # and the library's own kernel gives the same bits
    assert_bits_equal(got, ctx.unary(D.HARDSIGMOID, x, float(alpha), float(beta)), "module vs library")
    ctx.free(din), ctx.free(dout)


def test_module_dynamic_shared_memory(ctx, case, module):
    case("module kernel ahip_module_row_sum, 37 rows x 1000, 128 threads, 512 B shared")
    rng = np.random.default_rng(8)
    x = rng.integers(-8, 9, size=(37, 1000)).astype(np.float32)  # small integers: every order sums exactly
    din, dout = ctx.upload(x), ctx.alloc(37 * 4)
    ctx.launch(module, "ahip_module_row_sum", (37, 1, 1), (128, 1, 1),
               [ctypes.c_void_p(dout.ptr), ctypes.c_void_p(din.ptr), ctypes.c_uint32(1000)], shared_bytes=128 * 4)
    assert_bits_equal(ctx.download(dout, (37,)), x.sum(-1), "row sums")
    ctx.free(din), ctx.free(dout)


def test_module_errors_are_reported_not_raised_on_the_device(ctx, case, module, image):
    case("module error paths")
    dout = ctx.alloc(1024)
    args = [ctypes.c_void_p(dout.ptr), ctypes.c_void_p(dout.ptr), ctypes.c_float(1), ctypes.c_float(0), ctypes.c_uint64(4)]
    with pytest.raises(_lib.AltiusHipError) as e:
        ctx.launch(module, "no_such_kernel", (1, 1, 1), (64, 1, 1), args)
    assert e.value.code == _lib.ERR_ARG and "no_such_kernel" in e.value.message
    for grid, block in [((1, 1, 1), (2048, 1, 1)), ((1, 1, 1), (64, 32, 1)), ((0, 1, 1), (64, 1, 1)),
                        ((1, 1, 1), (0, 1, 1)), ((1, 70000, 1), (64, 1, 1))]:
        with pytest.raises(_lib.AltiusHipError) as e:
            ctx.launch(module, "ahip_module_hard_sigmoid", grid, block, args)
        assert e.value.code == _lib.ERR_ARG
    with pytest.raises(_lib.AltiusHipError) as e:
        ctx.launch(module, "ahip_module_row_sum", (1, 1, 1), (64, 1, 1), args[:3], shared_bytes=161 * 1024)
    assert e.value.code == _lib.ERR_ARG
    for bad in (b"", b"not a code object at all....", image[:4]):
        with pytest.raises(_lib.AltiusHipError) as e:
            ctx.load_module(bad)
        assert e.value.code == _lib.ERR_ARG
    # the context still works afterwards
    ctx.launch(module, "ahip_module_hard_sigmoid", (1, 1, 1), (64, 1, 1), args)
    ctx.sync()
    ctx.free(dout)

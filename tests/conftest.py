import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure): built on demand from oracle/."""
    import oracle as O

    O.lib()
    return O


@pytest.fixture(scope="session")
def ctx():
    """A device context on GPU 0 through the C ABI.  Fails loudly without the library."""
    from altius_amd import device

    c = device.Context(0)
    yield c
    c.close()


def announce(msg):
    """Names the case before it touches the GPU, so a faulting run still says which one it was."""
    print(f"[case] {msg}", flush=True)


@pytest.fixture
def case():
    return announce


# ---- comparison helpers -------------------------------------------------------

RTOL = 1e-5  # the parity bar: 1e-5 relative / 1e-6 absolute for fp32
ATOL = 1e-6


def assert_close(actual, expected, rtol=RTOL, atol=ATOL, what=""):
    actual = np.asarray(actual)
    expected = np.asarray(expected)
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    both_nan = np.isnan(actual) & np.isnan(expected)
    same_inf = np.isinf(actual) & np.isinf(expected) & (np.sign(actual) == np.sign(expected))
    with np.errstate(invalid="ignore"):
        err = np.abs(actual.astype(np.float64) - expected.astype(np.float64))
        ok = (err <= atol + rtol * np.abs(expected.astype(np.float64))) | both_nan | same_inf
    if not ok.all():
        bad = np.argwhere(~ok)
        i = tuple(bad[0])
        raise AssertionError(
            f"{what}: {len(bad)} of {actual.size} elements differ; first at {i}: "
            f"actual {actual[i]!r} expected {expected[i]!r}; max abs err {np.nanmax(np.where(ok, 0, err))}"
        )


def assert_bits_equal(actual, expected, what="", zero_sign_free=False):
    """Bit-for-bit equality of two float32 arrays (NaN payloads excepted); exact equality of
    values and element type for integer and bool arrays."""
    if np.asarray(expected).dtype.kind in "iub" or np.asarray(actual).dtype.kind in "iub":
        actual, expected = np.asarray(actual), np.asarray(expected)
        assert actual.dtype == expected.dtype, f"{what}: dtype {actual.dtype} vs {expected.dtype}"
        assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
        if not np.array_equal(actual, expected):
            bad = np.argwhere(actual != expected)
            i = tuple(bad[0])
            raise AssertionError(f"{what}: {len(bad)} of {actual.size} elements differ; first at {i}: {actual[i]} vs {expected[i]}")
        return
    actual = np.asarray(actual, dtype=np.float32, order="C")
    expected = np.asarray(expected, dtype=np.float32, order="C")
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    a = actual.view(np.uint32)
    e = expected.view(np.uint32)
    ok = (a == e) | (np.isnan(actual) & np.isnan(expected))
    if zero_sign_free:
        ok |= (actual == 0) & (expected == 0)
    if not ok.all():
        bad = np.argwhere(~ok)
        i = tuple(bad[0])
        raise AssertionError(
            f"{what}: {len(bad)} of {actual.size} elements differ in bits; first at {i}: "
            f"actual {actual[i]!r} (0x{a[i]:08x}) expected {expected[i]!r} (0x{e[i]:08x})"
        )

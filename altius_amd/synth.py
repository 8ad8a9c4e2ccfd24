"""Seeded synthetic inputs for the five benchmark configurations.

Counter-based (Philox) streams, one per tensor, so any tensor can be regenerated
on its own on any machine.  Shapes can be scaled down through `batch` for tests
that have to finish in seconds on a CPU.
"""
import numpy as np


def _rng(seed):
    return np.random.Generator(np.random.Philox(key=int(seed)))


def normal(seed, shape, mean=0.0, std=1.0):
    x = _rng(seed).standard_normal(size=shape, dtype=np.float32)
    if std != 1.0:
        x *= np.float32(std)
    if mean != 0.0:
        x += np.float32(mean)
    return x


def uniform(seed, shape):
    """U[0,1), the distribution the reference's own tests draw from."""
    return _rng(seed).random(size=shape, dtype=np.float32)


def attention_mask(seed, shape, p_masked=0.1, masked_value=-1e4):
    """0 where attended, masked_value where masked (Bernoulli(p_masked))."""
    u = _rng(seed).random(size=shape, dtype=np.float32)
    return np.where(u < p_masked, np.float32(masked_value), np.float32(0.0)).astype(np.float32)


# A divisor that is not a power of two, so Div is not an exponent shift.
DIV_SCALAR = np.float32(np.sqrt(np.float32(64.5)))
SQRT2 = np.float32(1.4142135)


def cfg0():
    """Add: A[1,197,768] + B[768]."""
    return {"a": normal(1000, (1, 197, 768)), "b": normal(1001, (768,))}


def cfg1(batch=8):
    """Softmax on [batch,12,197,197] * 0.125; LayerNorm on [batch,197,768]."""
    return {
        "scores": normal(1100, (batch, 12, 197, 197), std=0.125),
        "x": normal(1101, (batch, 197, 768)),
        "gamma": normal(1102, (768,), mean=1.0, std=0.02),
        "beta": normal(1103, (768,), mean=0.0, std=0.02),
        "eps": 1e-5,
    }


def cfg2(batch=32):
    """Unfused LayerNorm chain on [batch,197,768]."""
    return {
        "x": normal(1200, (batch, 197, 768)),
        "gamma": normal(1201, (768,), mean=1.0, std=0.02),
        "beta": normal(1202, (768,), mean=0.0, std=0.02),
        "two": np.float32(2.0),
        "eps": np.float32(1e-5),
    }


def cfg3(batch=32):
    """erf-GELU on [batch,197,3072]; squeeze-excite on NCHW [batch,576,7,7]."""
    return {
        "x": normal(1300, (batch, 197, 3072)),
        "se": normal(1301, (batch, 576, 7, 7)),
        "alpha": np.float32(1.0 / 6.0),
        "beta": np.float32(0.5),
        "sqrt2": SQRT2,
    }


def cfg4(batch=256):
    """Large-batch stress: masked Add + Softmax, axis-1 ReduceMax, scalar Div."""
    return {
        "scores": normal(1400, (batch, 12, 197, 197)),
        "mask": attention_mask(1401, (batch, 1, 1, 197)),
        "rmax_in": normal(1402, (batch, 768, 197)),
        "div_in": normal(1403, (batch, 197, 768)),
        "div_scalar": DIV_SCALAR,
    }

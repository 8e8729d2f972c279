"""Shared helpers of the tests: seeded inputs and the error measure."""
import contextlib
import os

import numpy as np
import torch


@contextlib.contextmanager
def knobs(**env):
    """Sets the library's tuning knobs (TL_* environment variables) for the block and has the library read
    them again (it reads the environment once per process otherwise); restores both on the way out."""
    from ternaryllm_amd import _lib
    old = {k: os.environ.get(k) for k in env}
    try:
        for k, v in env.items():
            os.environ[k] = str(v)
        _lib.lib().tl_reload_options()
        yield
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        _lib.lib().tl_reload_options()


def ternary_weight(K, N, sparsity, seed):
    """The reference's i.i.d. rule (TernaryLinear.py:79-83) on a seeded CPU generator -> int32 [K, N] numpy."""
    g = torch.Generator().manual_seed(seed)
    r = torch.rand((K, N), generator=g)
    w = torch.zeros((K, N), dtype=torch.int32)
    w[(r >= sparsity) & (r < (sparsity + 1) / 2)] = -1
    w[r >= (sparsity + 1) / 2] = 1
    return w.numpy()


def activations(M, K, seed, dtype=torch.float32, integer=False):
    """N(0,1) activations, or small integers (every partial sum is then exact in fp32, so any
    summation order must give bit-identical results -- the trick of the reference's own CPU checks,
    ternaryLLM_CPU/src/initData.hpp:18-28)."""
    g = torch.Generator().manual_seed(seed)
    if integer:
        x = torch.randint(-8, 9, (M, K), generator=g).to(torch.float32)
    else:
        x = torch.randn((M, K), generator=g)
    return x.to(dtype)


def max_rel_err(y, y_ref, x, w):
    """max |y - y_ref| / max(|y_ref|, ||x_row||_2 * sqrt(density)).

    The floor is the RMS magnitude an output of that row has for a weight of this density, so
    outputs that happen to cancel to ~0 are measured against the scale of their row instead of
    against themselves."""
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    x = np.asarray(x, dtype=np.float64)
    density = float(np.count_nonzero(w)) / w.size
    floor = np.linalg.norm(x, axis=1, keepdims=True) * np.sqrt(max(density, 1e-12))
    floor = np.maximum(floor, 1e-30)
    return float(np.max(np.abs(y - y_ref) / np.maximum(np.abs(y_ref), floor)))


FP32_TOL = 1e-5   # fp32 activations, fp32 accumulate, fp32 output
FP16_TOL = 2e-3   # fp16 activations, fp32 accumulate, fp16 output

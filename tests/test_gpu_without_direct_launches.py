"""The kernels that large launches use, on the small and ragged shapes of the primitive, collective and special-value suites.

Small launches normally take kernels of their own (addresses resolved on the host, a two-dimensional grid), so the
suites in test_gpu_primitives.py and test_gpu_collectives.py exercise those.  Here every test of those modules runs
once more with HcommGfxSetDirectLaunches(0): the same shapes, the same checks against the oracle, through k_copy,
k_reduce2, k_fold_chain(_small) and k_fold_tree."""
import functools

import pytest

import hcomm_amd as h
import test_gpu_collectives as collectives
import test_gpu_primitives as primitives
import test_gpu_special_values as special


pytestmark = pytest.mark.gpu


def without_direct_launches(fn):
    @functools.wraps(fn)  # keeps the marks (gpu, parametrize) and, through __wrapped__, the argument names
    def run(*args, **kwargs):
        before = h.HcommGfxSetDirectLaunches(0)
        try:
            return fn(*args, **kwargs)
        finally:
            h.HcommGfxSetDirectLaunches(before)
    return run


for _mod in (primitives, collectives, special):
    for _name in dir(_mod):
        _fn = getattr(_mod, _name)
        if _name.startswith("test_") and callable(_fn):
            globals()[f"{_name}__large_launch_kernels"] = without_direct_launches(_fn)

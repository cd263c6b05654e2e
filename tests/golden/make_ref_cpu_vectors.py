"""Writes tests/golden/ref_cpu_vectors.npz from the reference's own CPU reduce code.

Needs oracle/_ref/libhcomm_ref.so, i.e. the reference tree at build time (`make -C oracle`): that library is
the reference's test/hccl_vm/src/plugin/runner/runner_utils/hccl_task_reduce_process.cc and
.../ccu_executor/ccu_fp16.h compiled in place.  The vectors are data only: seeded inputs and what the
reference code returned for them.  Note the reference's Min / Max loops leave element 0 untouched.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
from util import gen  # noqa: E402


def main():
    R = oracle.ref()
    if R is None:
        sys.exit("oracle/_ref is not built")
    out = {}
    rng = np.random.default_rng(2024)
    x = (rng.standard_normal(4096) * np.exp2(rng.integers(-28, 18, 4096))).astype(np.float32)
    x[:8] = [0.0, -0.0, 65504.0, 65520.0, 2.0 ** -24, 2.0 ** -25, np.inf, -np.inf]
    h = np.empty(x.size, np.uint16)
    R.ref_fp16_from_float_n(x.ctypes.data, h.ctypes.data, x.size)
    out["f32_in"], out["f16_out"] = x, h
    for name, dt in (("i8", oracle.I8), ("i16", oracle.I16), ("i32", oracle.I32), ("f16", oracle.F16),
                     ("f32", oracle.F32)):
        d, s = gen(dt, 2048, 7, "wide"), gen(dt, 2048, 8, "wide")
        if dt == oracle.F16:
            d[(d & 0x7C00) == 0x7C00] = 0x3C00
            s[(s & 0x7C00) == 0x7C00] = 0xBC00
        if dt == oracle.F32:
            d, s = np.nan_to_num(d, nan=1.0, posinf=3e38, neginf=-3e38), np.nan_to_num(s, nan=2.0, posinf=3e38, neginf=-3e38)
        out[name + "_d"], out[name + "_s"] = d, s
        for tag, fn in (("sum", R.ref_mem_reduce_sum), ("min", R.ref_mem_reduce_min), ("max", R.ref_mem_reduce_max)):
            dd, ss = d.copy(), s.copy()
            fn(ss.ctypes.data, dd.ctypes.data, dd.nbytes, dt)
            out["%s_%s" % (name, tag)] = dd
    np.savez_compressed(os.path.join(HERE, "ref_cpu_vectors.npz"), **out)
    print("wrote ref_cpu_vectors.npz with", sorted(out))


if __name__ == "__main__":
    main()

"""Shared helpers of the test suite: seeded inputs in storage form, device upload / download, comparisons."""
import numpy as np

import oracle

DT = {"int8": oracle.I8, "int16": oracle.I16, "int32": oracle.I32, "fp16": oracle.F16, "fp32": oracle.F32,
      "bf16": oracle.BF16}
OPS = {"sum": oracle.SUM, "prod": oracle.PROD, "max": oracle.MAX, "min": oracle.MIN}
UNIT = {oracle.I8: 1, oracle.I16: 2, oracle.I32: 4, oracle.F16: 2, oracle.F32: 4, oracle.BF16: 2}


def f32_to_bf16_bits(x):
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def gen(dtype, count, seed, kind="default"):
    """Seeded input in storage form (16-bit floats as raw uint16).

    kind: default - the distribution the benchmark configs name for the type:
            fp32 uniform[-1,1), bf16 normal(0,1)*1e-3, fp16 uniform[-1,1), int32 ints in [-2^20, 2^20],
            int8 ints in [-8, 8], int16 ints in [-1000, 1000];
          prod - values close to 1 (fp: uniform[0.99,1.01]; ints: {-1, 1, 2} sparsely);
          wide - full range of the type (integers wrap, floats span many exponents);
          special - floating types only: signed zeros, infinities, quiet NaNs whose payload is taken from the seed,
            denormals, the largest finite values (see gen_special).
    """
    if kind == "special":
        return gen_special(dtype, count, seed)
    rng = np.random.default_rng(seed)
    if dtype == oracle.F32:
        if kind == "prod":
            return rng.uniform(0.99, 1.01, count).astype(np.float32)
        if kind == "wide":
            return (rng.standard_normal(count) * np.exp2(rng.integers(-40, 40, count))).astype(np.float32)
        return rng.uniform(-1.0, 1.0, count).astype(np.float32)
    if dtype == oracle.BF16:
        if kind == "prod":
            return f32_to_bf16_bits(rng.uniform(0.99, 1.01, count).astype(np.float32))
        if kind == "wide":
            return rng.integers(0, 1 << 16, count, dtype=np.uint32).astype(np.uint16)
        return f32_to_bf16_bits((rng.standard_normal(count) * 1e-3).astype(np.float32))
    if dtype == oracle.F16:
        if kind == "prod":
            return rng.uniform(0.99, 1.01, count).astype(np.float16).view(np.uint16)
        if kind == "wide":
            return rng.integers(0, 1 << 16, count, dtype=np.uint32).astype(np.uint16)
        return rng.uniform(-1.0, 1.0, count).astype(np.float16).view(np.uint16)
    info = {oracle.I8: (np.int8, 8), oracle.I16: (np.int16, 1000), oracle.I32: (np.int32, 1 << 20)}[dtype]
    if kind == "wide":
        ii = np.iinfo(info[0])
        return rng.integers(ii.min, ii.max + 1, count, dtype=np.int64).astype(info[0])
    if kind == "prod":
        return rng.choice(np.array([1, 1, 1, -1, 2], dtype=info[0]), count)
    return rng.integers(-info[1], info[1] + 1, count, dtype=np.int64).astype(info[0])


# per floating type: storage dtype, bit patterns of +0, +inf, largest finite, smallest and largest denormal, smallest
# normal, 1.0, a quiet NaN without payload, the sign bit, and how many payload bits lie below the quiet bit
_SPECIAL = {
    oracle.F32: (np.uint32, 0x00000000, 0x7F800000, 0x7F7FFFFF, 0x00000001, 0x007FFFFF, 0x00800000, 0x3F800000, 0x7FC00000,
                 0x80000000, 22),
    oracle.F16: (np.uint16, 0x0000, 0x7C00, 0x7BFF, 0x0001, 0x03FF, 0x0400, 0x3C00, 0x7E00, 0x8000, 9),
    oracle.BF16: (np.uint16, 0x0000, 0x7F80, 0x7F7F, 0x0001, 0x007F, 0x0080, 0x3F80, 0x7FC0, 0x8000, 6),
}


def gen_special(dtype, count, seed):
    """Inputs on which the operand roles of MAX / MIN decide the bits of the result (the reference keeps dst on a tie
    and on an unordered comparison, hccl_task_reduce_process.cc:36-40,50-54) and on which SUM / PROD overflow, cancel
    to NaN and pass through the denormal range.  Element i draws from the value set of zone i % 6:
      0  +0 and -0 only: every comparison along a chain or a tree is a tie;
      1  signed zeros and quiet NaNs: ties and unordered comparisons;
      2  infinities, the largest finite values, zeros, NaNs: inf - inf, 0 * inf, overflow;
      3  denormals, the smallest normal value, zeros;
      4  all of the above and +-1;
      5  the benign values of kind "default".
    Every NaN carries a payload derived from the seed (callers seed each rank differently), so that which operand's
    NaN survived shows in the bits."""
    bits, zero, inf, big, dmin, dmax, nmin, one, qnan, sign, pbits = _SPECIAL[dtype]
    rng = np.random.default_rng(seed + 77777)
    tag = 1 + seed % ((1 << pbits) - 1)
    both = lambda *v: [x for y in v for x in (y, y | sign)]
    zones = [both(zero), both(zero, zero, zero, qnan | tag), both(inf, big, zero, qnan | tag),
             both(dmin, dmax, nmin, zero), both(zero, inf, big, dmin, dmax, nmin, one, qnan | tag)]
    out = np.ascontiguousarray(gen(dtype, count, seed, "default")).view(bits).copy()
    for z, values in enumerate(zones):
        n = len(range(z, count, 6))
        out[z::6] = np.array(values, dtype=bits)[rng.integers(0, len(values), n)]
    return out.view(np.float32) if dtype == oracle.F32 else out


def to_dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).copy()).cuda()


def from_dev(t, like):
    return t.cpu().numpy().view(like.dtype).reshape(like.shape)


def is_float(dtype):
    return dtype in (oracle.F16, oracle.F32, oracle.BF16)


def assert_same(got, want, dtype, what="", nan_bits=False):
    """Bit-exact; for floating types two NaNs of any payload compare equal unless nan_bits is set (MAX and MIN move
    bit patterns, so there the payload and sign of a surviving NaN are part of the result)."""
    if got.dtype != want.dtype:
        got = got.view(want.dtype)
    if nan_bits:
        raw = {1: np.uint8, 2: np.uint16, 4: np.uint32}[want.dtype.itemsize]
        g, w = got.view(raw), want.view(raw)
        if np.array_equal(g, w):
            return
        bad = np.flatnonzero(g != w)
        i = int(bad[0])
        raise AssertionError("%s: %d of %d elements differ in their bits, first at %d: got %#x want %#x"
                             % (what, bad.size, g.size, i, int(g[i]), int(w[i])))
    if np.array_equal(got, want) if not is_float(dtype) else np.array_equal(got.view(np.uint8), want.view(np.uint8)):
        return
    if is_float(dtype):
        if dtype == oracle.F32:
            gn, wn = np.isnan(got), np.isnan(want)
            ok = (got.view(np.uint32) == want.view(np.uint32)) | (gn & wn)
        else:
            exp_mask, man_mask = (0x7C00, 0x03FF) if dtype == oracle.F16 else (0x7F80, 0x007F)
            gn = ((got & exp_mask) == exp_mask) & ((got & man_mask) != 0)
            wn = ((want & exp_mask) == exp_mask) & ((want & man_mask) != 0)
            ok = (got == want) | (gn & wn)
        if ok.all():
            return
        bad = np.flatnonzero(~ok)
    else:
        bad = np.flatnonzero(got != want)
    i = int(bad[0])
    raise AssertionError("%s: %d of %d elements differ, first at %d: got %r want %r"
                         % (what, bad.size, got.size, i, got[i], want[i]))

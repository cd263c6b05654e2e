"""Pins the element semantics of the CPU oracle (oracle/hcomm_oracle.c) against things it does not define
itself: numpy's typed arithmetic, IEEE binary16 as numpy implements it, torch.bfloat16, the reference's own
CPU reduce code compiled from its sources (oracle/_ref, when present) and vectors that code produced
(tests/golden/ref_cpu_vectors.npz)."""
import os

import numpy as np
import pytest

import oracle
from util import gen

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def np_op(d, s, op):
    """dst (op) src with the reference's tie rule, in numpy's own arithmetic of the array dtype."""
    with np.errstate(all="ignore"):
        if op == oracle.SUM:
            return d + s
        if op == oracle.PROD:
            return d * s
        if op == oracle.MAX:
            return np.where(s > d, s, d)
        return np.where(s < d, s, d)


# ---- integers: closed form, wrap-around ------------------------------------------------------------------

@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_int8_all_pairs(op):
    v = np.arange(-128, 128, dtype=np.int8)
    d, s = np.repeat(v, 256).copy(), np.tile(v, 256).copy()
    want = np_op(d, s, op).astype(np.int8)
    assert np.array_equal(oracle.reduce(d.copy(), s, oracle.I8, op), want)


@pytest.mark.parametrize("dt,npdt", [(oracle.I16, np.int16), (oracle.I32, np.int32)])
@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_int16_int32_wrap(dt, npdt, op):
    ii = np.iinfo(npdt)
    edge = np.array([ii.min, ii.min + 1, -1, 0, 1, ii.max - 1, ii.max, 12345, -12345], dtype=npdt)
    d = np.concatenate([np.repeat(edge, edge.size), gen(dt, 100000, 1, "wide")])
    s = np.concatenate([np.tile(edge, edge.size), gen(dt, 100000, 2, "wide")])
    want = np_op(d, s, op).astype(npdt)  # numpy integer arithmetic wraps modulo 2^bits
    assert np.array_equal(oracle.reduce(d.copy(), s, dt, op), want)


def test_known_answers_int():
    d = np.array([127, -128, 100, -100, 5], np.int8)
    s = np.array([1, -1, 100, -100, -7], np.int8)
    assert oracle.reduce(d.copy(), s, oracle.I8, oracle.SUM).tolist() == [-128, 127, -56, 56, -2]
    assert oracle.reduce(d.copy(), s, oracle.I8, oracle.PROD).tolist() == [127, -128, 16, 16, -35]
    assert oracle.reduce(d.copy(), s, oracle.I8, oracle.MAX).tolist() == [127, -1, 100, -100, 5]
    assert oracle.reduce(d.copy(), s, oracle.I8, oracle.MIN).tolist() == [1, -128, 100, -100, -7]


# ---- fp32: one IEEE operation -----------------------------------------------------------------------------

@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD, oracle.MAX, oracle.MIN])
def test_fp32_against_numpy(op):
    sp = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 1e-45, -1e-45, 1.17549435e-38, 3.4028235e38, -3.4028235e38,
                   1e8, 1.0000001], np.float32)
    d = np.concatenate([np.repeat(sp, sp.size), gen(oracle.F32, 200000, 3, "wide"), gen(oracle.F32, 1000, 5)])
    s = np.concatenate([np.tile(sp, sp.size), gen(oracle.F32, 200000, 4, "wide"), gen(oracle.F32, 1000, 6)])
    want = np_op(d, s, op).astype(np.float32)
    got = oracle.reduce(d.copy(), s, oracle.F32, op)
    both_nan = np.isnan(got) & np.isnan(want)
    assert ((got.view(np.uint32) == want.view(np.uint32)) | both_nan).all()


def test_fp_max_min_keep_dst_on_tie_and_nan():
    """(src > dst) ? src : dst - signed zeros tie, NaN compares false, so dst survives in both cases
    (llt_hccl_stub.cc:4089-4095 with src1 = src; hccl_task_reduce_process.cc:36-40,50-54)."""
    nan = np.float32(np.nan)
    d = np.array([0.0, -0.0, nan, 1.0, nan], np.float32)
    s = np.array([-0.0, 0.0, 1.0, nan, nan], np.float32)
    for op in (oracle.MAX, oracle.MIN):
        got = oracle.reduce(d.copy(), s, oracle.F32, op)
        assert got.view(np.uint32).tolist() == d.view(np.uint32).tolist()
    # same rule on the 16-bit types, on raw bit patterns
    for dt, pz, nz, qn, one in ((oracle.F16, 0x0000, 0x8000, 0x7E00, 0x3C00), (oracle.BF16, 0x0000, 0x8000, 0x7FC0, 0x3F80)):
        d16 = np.array([pz, nz, qn, one], np.uint16)
        s16 = np.array([nz, pz, one, qn], np.uint16)
        for op in (oracle.MAX, oracle.MIN):
            assert oracle.reduce(d16.copy(), s16, dt, op).tolist() == d16.tolist()


# ---- fp16 -------------------------------------------------------------------------------------------------

ALL16 = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)


def rounding_stress_f32():
    """float32 values around every fp16 rounding boundary + random wide values + overflow / underflow edges."""
    h = ALL16[(ALL16 & 0x7C00) != 0x7C00]            # finite halfs
    f = h.view(np.float16).astype(np.float32)
    nxt = (h + 1).astype(np.uint16)
    ok = (nxt & 0x7C00) != 0x7C00
    mid = ((f[ok].astype(np.float64) + nxt[ok].view(np.float16).astype(np.float64)) / 2).astype(np.float32)
    around = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])
    edges = np.array([65504.0, 65519.99, 65520.0, 65535.9, 65536.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                      2.0 ** -26, 5.96e-8, 0.0, np.inf], np.float32)
    rnd = np.random.default_rng(0)
    wide = (rnd.standard_normal(1 << 20) * np.exp2(rnd.integers(-30, 18, 1 << 20))).astype(np.float32)
    v = np.concatenate([f, around, edges, wide])
    return np.concatenate([v, -v])


def orc_to_f16(x):
    L = oracle.lib()
    return np.array([L.orc_f32_to_f16(float(v)) for v in x], np.uint16)


def test_fp16_to_fp32_exhaustive_vs_numpy():
    L = oracle.lib()
    got = np.array([L.orc_f16_to_f32(int(h)) for h in ALL16], np.float32)
    want = ALL16.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.isnan(got[nan]).all()


def test_fp32_to_fp16_rounding_vs_numpy_via_sum():
    """x + 0 through the oracle's fp16 SUM path = round-to-nearest-even conversion of every stress value:
    feed fp16 pairs whose exact fp32 sum hits the rounding boundaries."""
    x = rounding_stress_f32()
    x = x[np.isfinite(x)][: 1 << 19]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)          # numpy: IEEE round-to-nearest-even
    got = orc_to_f16(x)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("op", [oracle.SUM, oracle.PROD])
def test_fp16_arithmetic_vs_numpy(op):
    """Every fp16 pattern against 48 partners.  numpy's float16 arithmetic is the correctly rounded result,
    which is what widening to fp32, operating and rounding once delivers (24 >= 2*11 + 2)."""
    partners = np.concatenate([np.random.default_rng(1).integers(0, 1 << 16, 40, dtype=np.uint32).astype(np.uint16),
                               np.array([0x0000, 0x8000, 0x0001, 0x7BFF, 0xFBFF, 0x3C00, 0x7C00, 0xFC00], np.uint16)])
    d = np.tile(ALL16, partners.size)
    s = np.repeat(partners, ALL16.size)
    with np.errstate(all="ignore"):
        want = (np_op(d.view(np.float16), s.view(np.float16), op)).astype(np.float16).view(np.uint16)
    got = oracle.reduce(d.copy(), s, oracle.F16, op)
    wn = np.isnan(want.view(np.float16))
    gn = np.isnan(got.view(np.float16))
    assert np.array_equal(gn, wn)
    assert np.array_equal(got[~wn], want[~wn])
    # NaN results are canonical: sign | 0x7e00 (ccu_fp16.h:121)
    assert set(np.unique(got[gn] & 0x7FFF).tolist()) <= {0x7E00}


@pytest.mark.parametrize("op", [oracle.MAX, oracle.MIN])
def test_fp16_max_min_vs_numpy(op):
    d = np.tile(ALL16, 8)
    s = np.repeat(np.array([0x0000, 0x8000, 0x3C00, 0xBC00, 0x7C00, 0xFC00, 0x7E00, 0x0001], np.uint16), ALL16.size)
    fd, fs = d.view(np.float16), s.view(np.float16)
    with np.errstate(invalid="ignore"):
        take = (fs > fd) if op == oracle.MAX else (fs < fd)
    want = np.where(take, s, d)
    assert np.array_equal(oracle.reduce(d.copy(), s, oracle.F16, op), want)


# ---- the reference's own code -----------------------------------------------------------------------------

needs_ref = pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref was not built (no reference tree)")


@needs_ref
def test_fp16_conversions_equal_reference_FP16_class():
    R = oracle.ref()
    back = np.empty(ALL16.size, np.float32)
    R.ref_fp16_to_float_n(ALL16.ctypes.data, back.ctypes.data, ALL16.size)
    L = oracle.lib()
    mine = np.array([L.orc_f16_to_f32(int(h)) for h in ALL16], np.float32)
    finite = (ALL16 & 0x7C00) != 0x7C00
    assert np.array_equal(mine[finite].view(np.uint32), back[finite].view(np.uint32))
    # Quirk of the reference's half_to_float NOT copied: it has no case for exponent 31, so +-inf widen to
    # +-65536 and NaNs to finite values (ccu_fp16.h:102-111).  The oracle widens them to IEEE inf / NaN.
    assert back[0x7C00] == 65536.0 and back[0xFC00] == -65536.0
    assert np.isinf(mine[0x7C00]) and np.isnan(mine[0x7E00])
    x = np.ascontiguousarray(rounding_stress_f32()[: 1 << 19])
    x = np.concatenate([x, np.array([np.nan, -np.nan, np.inf, -np.inf], np.float32)])
    ref_h = np.empty(x.size, np.uint16)
    R.ref_fp16_from_float_n(x.ctypes.data, ref_h.ctypes.data, x.size)
    assert np.array_equal(orc_to_f16(x), ref_h)


@needs_ref
@pytest.mark.parametrize("dt", [oracle.I8, oracle.I16, oracle.I32, oracle.F16, oracle.F32])
def test_reduce_loops_equal_reference_MemReduce(dt):
    """MemReduceSum / Min / Max of the reference (hccl_task_reduce_process.cc:57-147), same inputs.
    The reference's Min / Max loops skip element 0 (:36,:50) - compared from element 1."""
    R = oracle.ref()
    n = 70001
    for kind in ("default", "wide"):
        d0, s0 = gen(dt, n, 21, kind), gen(dt, n, 22, kind)
        if dt == oracle.F16 and kind == "wide":  # keep NaN out: their sign/payload is not pinned by the reference
            d0[(d0 & 0x7C00) == 0x7C00] = 0x3C00
            s0[(s0 & 0x7C00) == 0x7C00] = 0xBC00
        if dt == oracle.F32 and kind == "wide":
            d0, s0 = np.nan_to_num(d0, nan=1.0), np.nan_to_num(s0, nan=2.0)
        nbytes = d0.nbytes
        for op, fn, first in ((oracle.SUM, R.ref_mem_reduce_sum, 0), (oracle.MIN, R.ref_mem_reduce_min, 1),
                              (oracle.MAX, R.ref_mem_reduce_max, 1)):
            ref_d, ref_s = d0.copy(), s0.copy()
            fn(ref_s.ctypes.data, ref_d.ctypes.data, nbytes, dt)
            mine = oracle.reduce(d0.copy(), s0.copy(), dt, op)
            a, b = mine[first:], ref_d[first:]
            if dt == oracle.F32:
                assert ((a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))).all(), (dt, op, kind)
            else:
                assert np.array_equal(a, b), (dt, op, kind)


def test_committed_reference_vectors():
    """Vectors written by tests/golden/make_ref_cpu_vectors.py from the compiled reference code."""
    z = np.load(os.path.join(GOLDEN, "ref_cpu_vectors.npz"))
    assert np.array_equal(orc_to_f16(z["f32_in"]), z["f16_out"])
    for name, dt in (("i8", oracle.I8), ("i16", oracle.I16), ("i32", oracle.I32), ("f16", oracle.F16),
                     ("f32", oracle.F32)):
        d, s = z[name + "_d"], z[name + "_s"]
        assert np.array_equal(oracle.reduce(d.copy(), s, dt, oracle.SUM).view(np.uint8), z[name + "_sum"].view(np.uint8))
        assert np.array_equal(oracle.reduce(d.copy(), s, dt, oracle.MAX)[1:].view(np.uint8),
                              z[name + "_max"][1:].view(np.uint8))
        assert np.array_equal(oracle.reduce(d.copy(), s, dt, oracle.MIN)[1:].view(np.uint8),
                              z[name + "_min"][1:].view(np.uint8))


# ---- bf16: no reference witness; pinned against torch only ----------------------------------------------

def test_bf16_against_torch():
    """PARITY UNPINNED against the reference (it has no bf16 arithmetic on any CPU path).  The oracle's
    definition - fp32 operation, round to nearest even - is checked against torch.bfloat16."""
    import torch
    L = oracle.lib()
    x = rounding_stress_f32()
    x = np.ascontiguousarray(x[np.isfinite(x)][: 1 << 18])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.orc_f32_to_bf16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)
    d, s = gen(oracle.BF16, 1 << 18, 1, "wide"), gen(oracle.BF16, 1 << 18, 2, "wide")
    for a in (d, s):  # keep NaN / inf out: torch's NaN payloads are its own
        a[(a & 0x7F80) == 0x7F80] = 0x3F80
    td = torch.from_numpy(d.view(np.int16)).view(torch.bfloat16)
    ts = torch.from_numpy(s.view(np.int16)).view(torch.bfloat16)
    for op, tw in ((oracle.SUM, td + ts), (oracle.PROD, td * ts)):
        want = tw.view(torch.int16).numpy().view(np.uint16)
        got = oracle.reduce(d.copy(), s, oracle.BF16, op)
        finite = (want & 0x7F80) != 0x7F80
        assert np.array_equal(got[finite], want[finite])
    assert L.orc_f32_to_bf16(float("nan")) & 0x7FFF == 0x7FC0


def test_dtype_sizes_match_size_table():
    """SIZE_TABLE, pkg_inc/legacy/hccl/dtype_common.h:18-36."""
    want = [1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1]
    assert [oracle.lib().orc_dtype_size(i) for i in range(18)] == want
    assert oracle.lib().orc_dtype_size(255) == 0


def test_special_inputs_make_roles_visible():
    """The inputs do what they are for: on them a MAX / MIN with the operands swapped leaves other bits, in every
    zone that holds ties or NaNs, for every floating type: what the GPU suite's special-value cases rely on."""
    for dtype, dt in (("fp32", oracle.F32), ("fp16", oracle.F16), ("bf16", oracle.BF16)):
        a, b = gen(dt, 6000, 1, "special"), gen(dt, 6000, 132, "special")
        for o in (oracle.MAX, oracle.MIN):
            d1, d2 = a.copy(), b.copy()
            oracle.reduce(d1, b.copy(), dt, o)   # a in the dst role
            oracle.reduce(d2, a.copy(), dt, o)   # b in the dst role
            raw = np.uint32 if dt == oracle.F32 else np.uint16
            differs = d1.view(raw) != d2.view(raw)
            for zone in (0, 1, 2, 4):
                assert differs[zone::6].sum() >= 50, (dtype, o, zone)

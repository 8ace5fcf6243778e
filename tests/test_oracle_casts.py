"""Pins for the C oracle's arithmetic: known answers, invariants, and torch's CPU casts."""

import numpy as np
import pytest
import torch

from oracle import c_oracle as co


def f32(x) -> int:
    return int(np.float32(x).view(np.uint32))


def test_bf16_known_answers():
    lib = co.lib()
    kat = {
        0x3F800000: 0x3F80,  # 1.0
        0x3F808000: 0x3F80,  # tie -> even (down)
        0x3F818000: 0x3F82,  # tie -> even (up)
        0x3F808001: 0x3F81,  # just above the tie
        0x3F807FFF: 0x3F80,  # just below the tie
        0x7F7FFFFF: 0x7F80,  # max float rounds to +inf
        0xFF7FFFFF: 0xFF80,
        0x00000000: 0x0000,
        0x80000000: 0x8000,  # -0 keeps its sign
        0x00008000: 0x0000,  # subnormal tie -> even
        0x00018000: 0x0002,
        0x7F800000: 0x7F80,
        0x7FC00001: 0x7FC0,  # NaN -> canonical quiet NaN
        0xFFFFFFFF: 0x7FC0,
        0x7F800001: 0x7FC0,  # signalling NaN too
    }
    for u, want in kat.items():
        assert lib.oracle_f32_to_bf16(u) == want, hex(u)


def test_bf16_round_trip_and_monotone():
    lib = co.lib()
    for h in range(0, 1 << 16):
        u = lib.oracle_bf16_to_f32(h)
        assert u == h << 16
        is_nan = (h & 0x7FFF) > 0x7F80
        assert lib.oracle_f32_to_bf16(u) == (0x7FC0 if is_nan else h)
    # positive floats are ordered like their bit patterns; rounding must be monotone
    us = np.sort(np.random.RandomState(0).randint(0, 0x7F800000, size=20000).astype(np.uint32))
    out = [lib.oracle_f32_to_bf16(int(u)) for u in us]
    assert all(a <= b for a, b in zip(out, out[1:]))


def test_bf16_matches_torch_cpu():
    rs = np.random.RandomState(1)
    u = rs.randint(0, 1 << 32, size=200000, dtype=np.uint64).astype(np.uint32)
    want = torch.from_numpy(u.view(np.float32).copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = co.cast(u, co.F32, co.BF16, np.uint16)
    nan = np.isnan(u.view(np.float32))
    assert np.array_equal(got[~nan], want[~nan])
    # NaN payloads are not pinned: ATen's vectorised CPU cast writes 0xFFFF, its scalar
    # c10::BFloat16 rule 0x7FC0 (the one restated here), CUDA's intrinsic 0x7FFF.  All are NaNs.
    assert np.all((got[nan] & 0x7FFF) > 0x7F80) and np.all((want[nan] & 0x7FFF) > 0x7F80)


def test_f16_known_answers():
    lib = co.lib()
    kat = {
        f32(1.0): 0x3C00,
        f32(-2.0): 0xC000,
        f32(65504.0): 0x7BFF,
        f32(65519.996): 0x7BFF,  # below the midpoint to 65536
        f32(65520.0): 0x7C00,  # the midpoint rounds to even = infinity
        f32(1e10): 0x7C00,
        f32(2.0**-24): 0x0001,  # smallest subnormal
        f32(2.0**-25): 0x0000,  # tie between 0 and the smallest subnormal -> even (0)
        f32(2.0**-25 * 1.0000001): 0x0001,
        f32(3 * 2.0**-25): 0x0002,  # tie between 1 and 2 ulp -> even
        f32(2.0**-14): 0x0400,  # smallest normal
        f32(2.0**-14 - 2.0**-25): 0x0400,  # rounds up across the subnormal/normal border
        f32(0.1): 0x2E66,
        f32(1.0 + 2.0**-11): 0x3C00,  # tie -> even
        f32(1.0 + 3 * 2.0**-11): 0x3C02,
        0x00000000: 0x0000,
        0x80000000: 0x8000,
        0x7F800000: 0x7C00,
        0xFF800000: 0xFC00,
    }
    for u, want in kat.items():
        assert lib.oracle_f32_to_f16(u) == want, hex(u)
    assert lib.oracle_f32_to_f16(0x7FC00000) & 0x7C00 == 0x7C00 and lib.oracle_f32_to_f16(0x7FC00000) & 0x3FF


def test_f16_round_trip_exhaustive_and_numpy():
    lib = co.lib()
    h = np.arange(1 << 16, dtype=np.uint16)
    want32 = h.view(np.float16).astype(np.float32).view(np.uint32)
    nan = np.isnan(h.view(np.float16))
    for i in range(1 << 16):
        u = lib.oracle_f16_to_f32(i)
        if nan[i]:
            assert (u & 0x7F800000) == 0x7F800000 and (u & 0x7FFFFF)
        else:
            assert u == int(want32[i])
            assert lib.oracle_f32_to_f16(u) == i
    rs = np.random.RandomState(2)
    u = rs.randint(0, 1 << 32, size=200000, dtype=np.uint64).astype(np.uint32)
    f = u.view(np.float32)
    keep = ~np.isnan(f)
    with np.errstate(over="ignore"):
        want = f[keep].astype(np.float16).view(np.uint16)
    got = co.cast(u[keep], co.F32, co.F16, np.uint16)
    assert np.array_equal(got, want)
    want_t = torch.from_numpy(f[keep].copy()).to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want_t)


@pytest.mark.parametrize("src,dst", [("f64", "bf16"), ("f64", "f16"), ("f64", "f32"), ("bf16", "f16"),
                                     ("f16", "bf16"), ("bf16", "f64"), ("f16", "f32"), ("f32", "f64")])
def test_other_casts_match_torch_cpu(src, dst):
    tt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "f64": torch.float64}
    code = {"f16": co.F16, "bf16": co.BF16, "f32": co.F32, "f64": co.F64}
    raw = {"f16": np.uint16, "bf16": np.uint16, "f32": np.uint32, "f64": np.uint64}
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(50000, generator=g, dtype=torch.float64) * torch.logspace(-12, 12, 50000, dtype=torch.float64))
    x = x.to(tt[src])
    want = x.to(tt[dst])
    bits_in = x.view({2: torch.int16, 4: torch.int32, 8: torch.int64}[x.element_size()]).numpy().view(raw[src])
    got = co.cast(bits_in, code[src], code[dst], raw[dst])
    want_bits = want.view({2: torch.int16, 4: torch.int32, 8: torch.int64}[want.element_size()]).numpy().view(raw[dst])
    assert np.array_equal(got, want_bits)


def test_gather_scatter_against_numpy():
    rs = np.random.RandomState(4)
    parent = rs.randint(0, 1 << 16, size=(5, 7, 12)).astype(np.uint16)
    view = parent.transpose(1, 0, 2)  # non-contiguous parent
    start, shape = (2, 1, 3), (4, 3, 6)
    strides = [s // 2 for s in view.strides]
    c = co.make_chunk(view.ctypes.data, start, shape, strides, co.B16, co.B16)
    out = np.zeros(shape, dtype=np.uint16)
    co.lib().oracle_gather(c, out.ctypes.data)
    want = view[2:6, 1:4, 3:9]
    assert np.array_equal(out, want)
    before = parent.copy()
    new = rs.randint(0, 1 << 16, size=shape).astype(np.uint16)
    co.lib().oracle_scatter(c, new.ctypes.data)
    expect = before.transpose(1, 0, 2).copy()
    expect[2:6, 1:4, 3:9] = new
    assert np.array_equal(parent.transpose(1, 0, 2), expect)  # nothing outside the slice moved


def test_reduce_is_fp32_rank_order():
    # (1 + 1e8) - 1e8 = 0 in fp32 but 1e8 - 1e8 + 1 = 1: the order of the peers is observable
    a = np.array([1.0, 1e8, 3.0], dtype=np.float32)
    b = np.array([1e8, -1e8, 4.0], dtype=np.float32)
    c_ = np.array([-1e8, 1.0, 5.0], dtype=np.float32)
    out = np.zeros(3, dtype=np.float32)
    scratch = np.zeros(3, dtype=np.float64)
    ch = co.make_chunk(0, (0,), (3,), (1,), co.F32, co.F32, peers=[a.ctypes.data, b.ctypes.data, c_.ctypes.data])
    assert co.lib().oracle_reduce(ch, out.ctypes.data, scratch.ctypes.data) == 0
    assert out.tolist() == [0.0, 1.0, 12.0]
    # bf16 partials: sum in fp32, one rounding at the end (256 + 1 + 1 = 258 exactly; bf16 steps of 2 there)
    parts = [np.array([v], dtype=np.float32) for v in (256.0, 1.0, 1.0)]
    pb = [co.cast(p.view(np.uint32), co.F32, co.BF16, np.uint16) for p in parts]
    ob = np.zeros(1, dtype=np.uint16)
    ch = co.make_chunk(0, (0,), (1,), (1,), co.BF16, co.BF16, peers=[p.ctypes.data for p in pb])
    assert co.lib().oracle_reduce(ch, ob.ctypes.data, scratch.ctypes.data) == 0
    assert int(ob[0]) == co.lib().oracle_f32_to_bf16(f32(258.0))  # a bf16-accumulated sum would give 256
    for op, want in (("avg", 86.0), ("max", 256.0), ("min", 1.0), ("product", 256.0)):
        ch = co.make_chunk(0, (0,), (1,), (1,), co.BF16, co.F32, peers=[p.ctypes.data for p in pb], op=op)
        of = np.zeros(1, dtype=np.float32)
        assert co.lib().oracle_reduce(ch, of.ctypes.data, scratch.ctypes.data) == 0
        assert of[0] == np.float32(want)


# ---- integers, bool and the 8-bit floats ------------------------------------------------------------------
_TORCH = {co.F16: torch.float16, co.BF16: torch.bfloat16, co.F32: torch.float32, co.F64: torch.float64, co.I8: torch.int8,
          co.U8: torch.uint8, co.I16: torch.int16, co.I32: torch.int32, co.I64: torch.int64, co.BOOL: torch.bool,
          co.F8E4M3: torch.float8_e4m3fn, co.F8E5M2: torch.float8_e5m2}
_RAW = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}
_NAMES = {"f16": co.F16, "bf16": co.BF16, "f32": co.F32, "f64": co.F64, "e4m3": co.F8E4M3, "e5m2": co.F8E5M2, "i8": co.I8,
          "u8": co.U8, "i16": co.I16, "i32": co.I32, "i64": co.I64, "bool": co.BOOL}


def _kats():
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cast_kats.json")) as f:
        return json.load(f)


def _from_hex(values, size):
    return np.array([int(v, 16) for v in values], dtype=np.uint64).astype(_RAW[size])


def _is_nan(raw, dt):
    t = torch.from_numpy(raw.view(np.uint8).copy()).view(_TORCH[dt])
    return torch.isnan(t.to(torch.float64) if dt != co.F64 else t).numpy()


@pytest.mark.parametrize("group", ["float_to_int", "float_to_float8", "int_to_float"])
def test_value_casts_known_answers(group):
    """Committed answers of torch's CPU ``Tensor.to`` for out-of-range floats, NaN into integers (what C++ leaves
    undefined) and the 8-bit float limits: truncation, INT_MIN for what does not fit, uint8 through int64."""
    for pair, kat in _kats()[group].items():
        s, d = (_NAMES[n] for n in pair.split("->"))
        src = _from_hex(kat["in"], co.lib().oracle_dtype_size(s))
        want = _from_hex(kat["out"], co.lib().oracle_dtype_size(d))
        got = co.cast(src, s, d, _RAW[co.lib().oracle_dtype_size(d)])
        differ = got != want
        if d in (co.F16, co.BF16, co.F32, co.F64, co.F8E4M3, co.F8E5M2):
            differ &= ~(_is_nan(got, d) & _is_nan(want, d))  # NaN payloads are not pinned
        assert not differ.any(), (pair, [kat["in"][i] for i in np.nonzero(differ)[0][:5]])


def test_float8_to_f32_every_pattern():
    for name, want in _kats()["float8_to_f32"].items():
        dt = _NAMES[name]
        got = co.cast(np.arange(256, dtype=np.uint8), dt, co.F32, np.uint32)
        want = _from_hex(want, 4)
        nan = _is_nan(want, co.F32)
        assert np.array_equal(got[~nan], want[~nan]) and _is_nan(got, co.F32)[nan].all(), name
        # and back: every finite pattern survives the round trip
        back = co.cast(got, co.F32, dt, np.uint8)
        assert np.array_equal(back[~nan], np.arange(256, dtype=np.uint8)[~nan])


def test_float8_rounding_is_to_nearest_even_and_monotone():
    """Independent of torch: every fp32 between two neighbouring 8-bit floats goes to the nearer one, ties to the
    even one; the mapping is monotone over the finite range."""
    for dt in (co.F8E4M3, co.F8E5M2):
        vals = co.cast(np.arange(128, dtype=np.uint8), dt, co.F32, np.uint32).view(np.float32).astype(np.float64)
        finite = np.isfinite(vals)
        codes = np.arange(128)[finite]
        vals = vals[finite]
        for lo, hi, c_lo, c_hi in zip(vals[:-1], vals[1:], codes[:-1], codes[1:]):
            mid = (lo + hi) / 2
            for x, want in ((lo + (hi - lo) * 0.49, c_lo), (lo + (hi - lo) * 0.51, c_hi), (mid, c_lo if c_lo % 2 == 0 else c_hi)):
                got = co.cast(np.array([np.float32(x)]).view(np.uint32), co.F32, dt, np.uint8)[0]
                assert got == want, (dt, x, got, want)
        xs = np.sort(np.random.RandomState(3).uniform(0, float(vals.max()), size=5000).astype(np.float32))
        out = co.cast(xs.view(np.uint32), co.F32, dt, np.uint8)
        assert np.all(np.diff(out.astype(np.int32)) >= 0)


def test_every_value_cast_matches_torch_cpu():
    """All 132 pairs of the twelve value types on random bit patterns and a spread of magnitudes, against torch's CPU
    ``Tensor.to`` (the call the reference makes, ir.py:125-126,137-138)."""
    g = torch.Generator().manual_seed(0)
    for s, sdt in _TORCH.items():
        raw = torch.randint(0, 256, (4000 * sdt.itemsize,), generator=g, dtype=torch.uint8)
        x = (raw % 2).view(sdt) if sdt == torch.bool else raw.view(sdt)
        if sdt.is_floating_point:
            x = torch.cat([x, (torch.randn(3000, generator=g, dtype=torch.float64) * 300).to(sdt),
                           (torch.randn(1000, generator=g, dtype=torch.float64) * 3e9).to(sdt)])
        src = x.view(torch.uint8).numpy().view(_RAW[sdt.itemsize])
        for d, ddt in _TORCH.items():
            if s == d:
                continue
            want = x.to(ddt).view(torch.uint8).numpy().view(_RAW[ddt.itemsize])
            got = co.cast(src, s, d, _RAW[ddt.itemsize])
            differ = got != want
            if ddt.is_floating_point:
                differ &= ~(_is_nan(got, d) & _is_nan(want, d))
            assert not differ.any(), (sdt, ddt, int(differ.sum()))

"""Writes tests/golden/cast_kats.json: known answers of ``Tensor.to(dtype)`` for the conversions whose result C++
leaves undefined (a float that does not fit the integer type, NaN into an integer) and for the 8-bit floats.

The values are what torch's own CPU kernels return in this environment (torch 2.10, x86-64, AVX-512; the
reference computes these casts with exactly that call, ``src/etha/comm/ir.py:125-126,137-138``).  Only torch is
run here; nothing of the reference is imported.  Inputs are stored as raw bit patterns (hex), outputs as
raw bit patterns as well.
"""

import json
import os

import torch

FLOATS = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "f64": torch.float64,
          "e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}
INTS = {"i8": torch.int8, "u8": torch.uint8, "i16": torch.int16, "i32": torch.int32, "i64": torch.int64, "bool": torch.bool}
RAW = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}

SPECIALS = [0.0, -0.0, 0.5, -0.5, 1.5, -1.5, 2.5, 127.0, 127.9, 128.0, 255.0, 255.9, 256.0, 300.0, -1.0, -128.0, -129.0, 32767.0,
            32768.0, 65535.0, 65536.0, -32769.0, 2147483520.0, 2147483647.0, 2147483648.0, -2147483648.0, -2147483649.0,
            -2147483904.0, 3e9, -3e9, 24812057633.7, 9.2e18, 9223372036854775807.0, 9.3e18, -9.3e18, 1e30, -1e30,
            float("inf"), -float("inf"), float("nan"),
            # around the 8-bit float limits and their subnormal ranges
            448.0, 464.0, 479.9, 480.0, 57344.0, 61440.0, 65520.0, 2.0 ** -6, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10,
            2.0 ** -14, 2.0 ** -16, 2.0 ** -17, 1.5 * 2.0 ** -17, 0.3, 0.0625, 17.0, 18.0, 19.0, 0.01171875]


def raw_hex(t):
    width = t.element_size() * 2
    mask = (1 << (8 * t.element_size())) - 1
    return [format(int(v) & mask, f"0{width}x") for v in t.contiguous().view(RAW[t.element_size()]).tolist()]


def main():
    out = {"float_to_int": {}, "float_to_float8": {}, "float8_to_f32": {}, "int_to_float": {}}
    for sname, sdt in FLOATS.items():
        x = torch.tensor(SPECIALS, dtype=torch.float64).to(sdt)
        for dname, ddt in INTS.items():
            out["float_to_int"][f"{sname}->{dname}"] = {"in": raw_hex(x), "out": raw_hex(x.to(ddt).view(torch.uint8) if ddt == torch.bool else x.to(ddt))}
        if sname not in ("e4m3", "e5m2"):
            for dname in ("e4m3", "e5m2"):
                out["float_to_float8"][f"{sname}->{dname}"] = {"in": raw_hex(x), "out": raw_hex(x.to(FLOATS[dname]).view(torch.uint8))}
    for name in ("e4m3", "e5m2"):
        every = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(FLOATS[name])
        out["float8_to_f32"][name] = raw_hex(every.to(torch.float32))
    ints = [0, 1, -1, 127, -128, 255, 256, 32767, -32768, 65535, 16777216, 16777217, 16777219, 2147483647, -2147483648,
            4294967295, 9007199254740993, 9223372036854775807, -9223372036854775808, 1234567890123456789]
    x = torch.tensor(ints, dtype=torch.int64)
    for dname, ddt in FLOATS.items():
        out["int_to_float"][f"i64->{dname}"] = {"in": raw_hex(x), "out": raw_hex(x.to(ddt).view(torch.uint8) if ddt.itemsize == 1 else x.to(ddt))}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cast_kats.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=0, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Writes tests/golden/packing_kat.json: known-answer vectors for the two row-major word orders.

Nothing here imports the oracle, the package or the reference.  Every expected word is derived from
the definition alone, one element at a time: element k of a 32-group is -1  <=>  bit p(k) is set,
with p(k) = k for `lsb_first` and p(k) = 15 - k//2 + 16*(k%2) for `half2` (the bit tables at
src/nanoquant/kernel/utils.py:99-104 of the reference; +1 -> 0 and -1 -> 1 at :95-96; column padding
is +1 at :87-93).  The hand-derived cases listed in the comments can be checked by eye.
"""
import json
import os
import random


def p(k, method):
    return k if method == "lsb_first" else 15 - k // 2 + 16 * (k % 2)


def pack_row(signs, method):
    words = []
    for w0 in range(0, len(signs), 32):
        group = signs[w0:w0 + 32]
        group = group + [1] * (32 - len(group))          # pad with +1
        word = 0
        for k, s in enumerate(group):
            if s == -1:
                word |= 1 << p(k, method)
        words.append(word - (1 << 32) if word >= (1 << 31) else word)   # as int32
    return words


def case(name, rows, note=""):
    return {"name": name, "note": note, "signs": rows,
            "lsb_first": [pack_row(r, "lsb_first") for r in rows],
            "half2": [pack_row(r, "half2") for r in rows]}


def one_minus(idx, n=32):
    return [[-1 if i == idx else 1 for i in range(n)]]


cases = [
    case("all_plus", [[1] * 32], "all +1 -> 0x00000000 in both orders"),
    case("all_minus", [[-1] * 32], "all -1 -> 0xFFFFFFFF = int32 -1 in both orders"),
    case("only_elem0", one_minus(0), "lsb_first 0x00000001; half2 0x00008000"),
    case("only_elem1", one_minus(1), "lsb_first 0x00000002; half2 0x80000000 = int32 -2147483648"),
    case("only_elem2", one_minus(2), "lsb_first 0x00000004; half2 0x00004000"),
    case("only_elem30", one_minus(30), "lsb_first 0x40000000; half2 0x00000001"),
    case("only_elem31", one_minus(31), "lsb_first 0x80000000; half2 0x00010000"),
    case("cols40_all_minus", [[-1] * 40], "two words; second has 8 real bits, 24 pad bits = 0: "
                                          "lsb_first [-1, 0xFF]; half2 [-1, 0xF000F000]"),
    case("alternating", [[1 if i % 2 == 0 else -1 for i in range(64)]],
         "odd elements -1: lsb_first 0xAAAAAAAA; half2 0xFFFF0000"),
]
for k in range(32):
    cases.append(case(f"walk_{k}", one_minus(k), "single -1 walking through the group"))

rng = random.Random(20260101)
for (r, c) in [(3, 32), (5, 96), (4, 100), (2, 7), (6, 257)]:
    rows = [[rng.choice((-1, 1)) for _ in range(c)] for _ in range(r)]
    cases.append(case(f"random_{r}x{c}", rows, "seeded random signs, ragged columns included"))

# eye-checkable constants
checks = {c["name"]: c for c in cases}
u32 = lambda v: v & 0xFFFFFFFF
assert u32(checks["only_elem0"]["half2"][0][0]) == 0x00008000
assert u32(checks["only_elem1"]["half2"][0][0]) == 0x80000000
assert u32(checks["only_elem31"]["half2"][0][0]) == 0x00010000
assert u32(checks["only_elem31"]["lsb_first"][0][0]) == 0x80000000
assert [u32(v) for v in checks["cols40_all_minus"]["half2"][0]] == [0xFFFFFFFF, 0xF000F000]
assert [u32(v) for v in checks["cols40_all_minus"]["lsb_first"][0]] == [0xFFFFFFFF, 0x000000FF]
assert u32(checks["alternating"]["half2"][0][0]) == 0xFFFF0000
assert u32(checks["alternating"]["lsb_first"][0][0]) == 0xAAAAAAAA

out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "packing_kat.json")
with open(out, "w") as f:
    json.dump({"cases": cases}, f, separators=(",", ":"))
print(out, os.path.getsize(out), "bytes,", len(cases), "cases")

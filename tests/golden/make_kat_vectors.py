"""Writes tests/golden/kat_vectors.json: known-answer vectors for the PolarQuant encode / pack /
dequant path, derived in EXACT rational arithmetic from the closed form of the transform, without
importing the oracle, the library or the reference.

What the mathematics fixes (the statements the vectors rest on):
  * the raw butterfly of rotation.py:22-32 is multiplication by the Sylvester Hadamard matrix
    H[j][k] = (-1)^popcount(j & k);
  * quantize (quantizer.py:85-106) compares  H (x * signs) / ||x||  with the midpoints of the
    literal centroid table (quantizer.py:27-35, 41-44), strictly:  idx = #{b : value > b};
  * pack (packing.py:20-55) puts element e into word e // vpw at bit (e % vpw) * bits,
    vpw = 32 // bits;
  * dequantize (quantizer.py:118-132) returns  norm * signs * (H c[idx]) / d.

The inputs are sparse vectors with small-integer entries whose norm is an exact float (3-4-5
triangles, four equal entries, ...), so every transformed value is a small rational that lies far
(more than 0.01, against a float32 error of about 1e-6) from every decision boundary — except the cases named "...on_boundary", where a value is exactly 0
and the strict comparison must put it in the lower bin.  A dropped or transposed stage, a wrong
sign placement, a non-strict comparison, a wrong field order in a word or a wrong dequant scale
changes the expected output of at least one vector.

Run:  python tests/golden/make_kat_vectors.py   (rewrites the JSON next to this file)
"""
import json
import os
from fractions import Fraction

CODEBOOKS = {      # literal tables of quantizer.py:27-35 (data)
    2: ["-1.5104", "-0.4528", "0.4528", "1.5104"],
    3: ["-2.1520", "-1.3440", "-0.7560", "-0.2451", "0.2451", "0.7560", "1.3440", "2.1520"],
    4: ["-2.7326", "-2.0690", "-1.6180", "-1.2562", "-0.9423", "-0.6568", "-0.3881", "-0.1284",
        "0.1284", "0.3881", "0.6568", "0.9423", "1.2562", "1.6180", "2.0690", "2.7326"],
}


def lcg_signs(d, seed):
    """A +-1 pattern from a 32-bit LCG (any fixed pattern serves: signs are an input of the path)."""
    out, s = [], seed & 0xFFFFFFFF
    for _ in range(d):
        s = (1664525 * s + 1013904223) & 0xFFFFFFFF
        out.append(1 if (s >> 31) else -1)
    return out


def popcount(v):
    return bin(v).count("1")


def case(name, d, bits, entries, norm, signs):
    """entries: {index: integer value}; norm: exact Fraction equal to the Euclidean norm."""
    assert sum(v * v for v in entries.values()) == norm * norm, name
    cb = [Fraction(c) for c in CODEBOOKS[bits]]
    bounds = [(cb[i] + cb[i + 1]) / 2 for i in range(len(cb) - 1)]
    x = [0] * d
    for i, v in entries.items():
        x[i] = v
    # value compared with the boundaries: raw butterfly of the unit vector (the 1/sqrt(d) of the
    # transform and the division by scale = 1/sqrt(d) cancel)
    idx, on_boundary = [], 0
    for k in range(d):
        w = sum(Fraction(v * signs[i] * (-1) ** popcount(i & k)) for i, v in entries.items())
        w = w / norm if norm else Fraction(0)
        margin = min(abs(w - b) for b in bounds)
        if margin == 0:
            on_boundary += 1
        else:
            assert margin > Fraction(1, 100), (name, k, float(w))     # far from every boundary (float32 error is ~1e-6)
        idx.append(sum(1 for b in bounds if w > b))
    vpw = 32 // bits
    words = [0] * ((d + vpw - 1) // vpw)
    for e, i in enumerate(idx):
        words[e // vpw] |= i << ((e % vpw) * bits)
    # dequant in exact arithmetic: norm * signs[e] * sum_k H[e][k] c[idx[k]] / d
    deq = []
    for e in range(d):
        acc = sum(cb[idx[k]] * (-1) ** popcount(e & k) for k in range(d))
        deq.append(float(norm * signs[e] * acc / d))
    return {"name": name, "dim": d, "bits": bits, "x": [float(v) for v in x], "signs": [float(s) for s in signs],
            "norm": float(norm), "idx": idx, "packed_hex": ["%08X" % w for w in words], "dequant": deq,
            "values_on_a_boundary": on_boundary}


def main():
    ones128 = [1] * 128
    s128 = lcg_signs(128, 2024)
    s64 = lcg_signs(64, 7)
    s32 = lcg_signs(32, 99)
    cases = [
        case("zero_vector", 128, 3, {}, Fraction(0), ones128),
        case("one_hot_j5_plain_signs", 128, 3, {5: 3}, Fraction(3), ones128),
        case("one_hot_j77_lcg_signs", 128, 3, {77: 2}, Fraction(2), s128),
        case("negative_one_hot_j127", 128, 3, {127: -4}, Fraction(4), s128),
        case("three_four_five", 128, 3, {3: 3, 96: 4}, Fraction(5), s128),
        case("three_four_five_mixed_sign", 128, 3, {64: -3, 1: 4}, Fraction(5), ones128),
        case("four_equal_entries_on_boundary", 128, 3, {0: 1, 17: 1, 34: 1, 127: 1}, Fraction(2), s128),
        case("six_eight_ten_d32_2bit", 32, 2, {4: 6, 9: 8}, Fraction(10), s32),
        case("four_equal_entries_on_boundary_d32_2bit", 32, 2, {1: 3, 2: -3, 12: 3, 31: 3}, Fraction(6), s32),
        case("one_hot_d64_4bit", 64, 4, {33: 5}, Fraction(5), s64),
        case("five_twelve_thirteen_d64_4bit", 64, 4, {2: 5, 63: -12}, Fraction(13), s64),
        case("one_hot_d32_3bit", 32, 3, {31: 7}, Fraction(7), s32),
    ]
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat_vectors.json")
    with open(out, "w") as f:
        json.dump({"about": "closed-form known answers; see make_kat_vectors.py", "cases": cases}, f, indent=1)
    print(f"wrote {len(cases)} cases to {out}")


if __name__ == "__main__":
    main()

"""Writes tests/golden/hash_kat.json: known answers for the count-sketch hash.

The values come from a second, independent statement of the ten lines at
communication/compressors/CountSketch.py:7-18, done with Python's unbounded
integers and explicit two's-complement helpers (no fixed-width integer type is
involved), so a slip in the C oracle's casts or shifts shows up as a mismatch.
Run:  python tests/golden/make_golden.py
"""
import json
import os

MASK = (1 << 32) - 1


def to_signed(u):
    u &= MASK
    return u - (1 << 32) if u >> 31 else u


def sar(s, k):
    """Arithmetic shift right of a signed 32-bit value (Python's >> on a negative int floors)."""
    return s >> k


def mix(value, a, b):
    h = to_signed(a * value + b)            # int h = a*value + b  (wraps)
    h = to_signed((h & MASK) ^ (sar(h, 16) & MASK))
    h = to_signed((h & MASK) * 0x85EBCA6B)  # unsigned multiply, reinterpret as int
    h = to_signed((h & MASK) ^ (sar(h, 13) & MASK))
    h = to_signed((h & MASK) * 0xC2B2AE35)
    h = to_signed((h & MASK) ^ (sar(h, 16) & MASK))
    return h


def c_mod(h, w):
    """C's truncating % for int operands."""
    q = abs(h) // w
    return h - (q if h >= 0 else -q) * w


def main():
    a, b = 994443, 609478
    seeds = {"cs": (a, b), "cs_sign": (a + 2, b + 3),
             "h3_1": (4113759, 2949676), "h3_1_sign": (4113759 + 4, 2949676 + 5),
             "h3_2": (9171025, 2171464), "h3_2_sign_update": (9171025 + 8, 2171464 + 4),
             "h3_2_sign_query": (9171025 + 8, 2171464 + 7)}
    values = list(range(0, 16)) + [255, 256, 1023, 5759, 65535, 65536, 1299999, 6499999,
                                   (1 << 31) - 1, 123456789]
    widths = [1, 2, 3, 65, 102, 409, 1152, 130000]
    out = {"values": values, "widths": widths, "seeds": {}}
    for name, (sa, sb) in seeds.items():
        pre = [mix(v, sa, sb) for v in values]
        out["seeds"][name] = {
            "a": sa, "b": sb, "mix": pre,
            "mod": {str(w): [c_mod(h, w) for h in pre] for w in widths},
        }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hash_kat.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()

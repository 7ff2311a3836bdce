"""Writes tests/golden/shuffle_orders.json: visiting orders of the reference's shuffled data
iterator (SelfOrganizingMapLib/DataIteratorShuffled.h), taken from the reference itself through
oracle/_ref (built from the reference's sources by oracle/Makefile).  Run where the reference
tree is present:  python tests/golden/make_shuffle_vectors.py
Short orders are stored whole; long ones as their first 16 entries and a CRC-32 of the
little-endian uint32 array."""
import json
import os
import sys
import zlib

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
import oracle as O  # noqa: E402

CASES = [(2, 2), (1234, 10), (1235, 10), (0, 7), (1234, 64), (42, 101), (2147483647, 100), (2 ** 40 + 3, 1000),
         (1234, 2000), (1234, 60000), (99, 65536), (99, 65537), (5, 70000)]


def main():
    if O.ref() is None:
        raise SystemExit("oracle/_ref is not built (the reference tree is needed)")
    out = []
    for seed, n in CASES:
        order = O.ref_shuffled_order(seed, n)
        entry = {"seed": seed, "n": n, "crc32": zlib.crc32(order.astype("<u4").tobytes())}
        entry["order" if n <= 128 else "head"] = order[: n if n <= 128 else 16].tolist()
        out.append(entry)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "shuffle_orders.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=0)
        f.write("\n")
    print("wrote", path, len(out), "cases")


if __name__ == "__main__":
    main()

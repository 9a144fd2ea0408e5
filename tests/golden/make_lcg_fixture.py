"""Writes tests/golden/lcg_pattern.json: known answers of the reference's
benchmark data pattern (example/bm/BmBenchmark/band_width_calculator.cpp:47-63),
worked out here with Python integers from the recurrence as published there:
    base_0 = rank;  base_{i+1} = (23 * base_i + 17) mod 32767
    word_i = -base_{i+1} if (i + rank) mod 3 == 0 else base_{i+1}
Run from the repository root:  python tests/golden/make_lcg_fixture.py"""

import json
import os

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lcg_pattern.json")


def pattern(rank, words):
    base = rank
    out = []
    for i in range(words):
        base = (base * 23 + 17) % 32767
        out.append(-base if (i + rank) % 3 == 0 else base)
    return out


if __name__ == "__main__":
    data = {"words": 24, "ranks": {str(r): pattern(r, 24) for r in (0, 1, 2, 7)}}
    # checksums over a longer run pin the tail of the sequence too
    data["sum_4096"] = {str(r): sum(pattern(r, 4096)) for r in (0, 1, 2, 7)}
    with open(OUT, "w") as f:
        json.dump(data, f, indent=1)
    print("wrote", OUT)

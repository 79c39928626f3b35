"""Writes tests/golden/hand_traced.json: known answers worked out by hand from the text of the
reference (it ships no fixtures of its own for this path; nothing of the reference is run here).

  orders     make_n_m(n, m) traced through the recursion of grouped_nm_tensor.py:37-50
  tiles      merged tiles [c][g][m] pushed by hand through the sort-and-scan of
             grouped_nm_tensor.py:255-297 (scores, descending sort with ties on larger column then
             larger pattern, acceptance scan)

Run from the repository root:  python tests/golden/make_hand_traced.py
"""
import json
import os

ORDERS = {
    "2:4": [[0, 1], [0, 2], [1, 2], [1, 3], [0, 3], [2, 3]],
    "1:8": [[5], [3], [1], [0], [2], [4], [6], [7]],
    "1:4": [[1], [0], [2], [3]],
    "1:2": [[0], [1]],
    "2:3": [[0, 1], [0, 2], [1, 2]],
    "1:3": [[0], [1], [2]],
    "2:2": [[0, 1]],
    "3:4": [[0, 1, 2], [0, 1, 3], [0, 2, 3], [1, 2, 3]],
}

TILES = [
    {   # 1:2, g = 1: two columns; every column gets its own best pattern
        "n": 1, "m": 2, "g": 1,
        "tile": [[[3.0, 1.0]], [[2.0, 5.0]]],
        "sorted": "(5,o1,p1) (3,o0,p0) (2,o1,p0) (1,o0,p1)",
        "idx": [0, 1], "val": [[3.0], [5.0]],
    },
    {   # capacity conflict: (3,o0,p0) is rejected because pattern 0 is already full
        "n": 1, "m": 2, "g": 1,
        "tile": [[[3.0, 1.0]], [[4.0, 0.5]]],
        "sorted": "(4,o1,p0) (3,o0,p0) (1,o0,p1) (0.5,o1,p1)",
        "idx": [1, 0], "val": [[4.0], [1.0]],
    },
    {   # all-zero 2:4 tile, g = 2: ties only, larger column first then larger pattern
        "n": 2, "m": 4, "g": 2,
        "tile": [[[0.0] * 4, [0.0] * 4] for _ in range(6)],
        "sorted": "all scores 0: (o11,p5) (o11,p4) ... the last pattern fills first with the last columns",
        "idx": [1, 0, 3, 2, 5, 4, 7, 6, 9, 8, 11, 10], "val": [[0.0, 0.0]] * 12,
    },
    {   # 2:2 (one pattern), g = 3: columns sorted by |a|+|b| descending, equal sums: larger column first
        "n": 2, "m": 2, "g": 3,
        "tile": [[[1.0, -1.0], [0.5, 4.0], [-2.0, 0.0]]],
        "sorted": "(4.5,o1) (2,o2) (2,o0)",
        "idx": [1, 2, 0], "val": [[0.5, 4.0], [-2.0, 0.0], [1.0, -1.0]],
    },
]

if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hand_traced.json")
    with open(out, "w") as f:
        json.dump({"orders": ORDERS, "tiles": TILES}, f, indent=1)
    print("wrote", out)

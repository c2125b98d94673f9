"""Writes the small fixtures of this directory.

``reference_test_counts.json``: the 500 group sizes that the reference's own test
draws (``test/test_scatter.py:8,11-13,18``: ``np.random.seed(0)`` then
``np.random.randint(100, 5000)`` once per group).  Stored so the closed-form
known-answer test does not depend on numpy's generator staying bit-stable.

``hand_cases.json`` is written by hand (tiny inputs with the expected outputs
worked out on paper from the reference kernels' text); this script only checks
that it parses.
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    np.random.seed(0)
    counts = [int(np.random.randint(100, 5000)) for _ in range(500)]
    with open(os.path.join(HERE, "reference_test_counts.json"), "w") as f:
        json.dump({"source": "np.random.seed(0); randint(100, 5000) x 500",
                   "num_total": int(sum(counts)), "max_cnt": int(max(counts)),
                   "counts": counts}, f)
    with open(os.path.join(HERE, "hand_cases.json")) as f:
        cases = json.load(f)
    print(len(counts), sum(counts), max(counts), min(counts), len(cases["cases"]))


if __name__ == "__main__":
    main()

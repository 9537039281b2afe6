"""Writes ``known_answers.json``: Newton-Schulz results that follow from scalar arithmetic alone.

For ``x = P diag(s) Q^T`` with P, Q (partial) permutation matrices, every matrix product of the iteration
keeps that structure, so the exact result is ``P diag(p_k(...p_1(s / ||s||_2))) Q^T`` where
``p(t) = a t + b t^3 + c t^5``.  Only Python floats are used here -- no matrix code, no oracle, no reference
import -- which makes these vectors an independent check of both the CPU oracle and the GPU kernels.

Run from the repository root:  python tests/golden/make_known_answers.py
"""

import json
import math
import os
import random

# Same literals as the published tables (three families are enough to exercise cycle / repeat_last / cubic).
TABLES = {
    "simple": ([(3.4445, -4.7750, 2.0315)], "cycle"),
    "quintic": (
        [
            (4.0848, -6.8946, 2.9270),
            (3.9505, -6.3029, 2.6377),
            (3.7418, -5.5913, 2.3037),
            (2.8769, -3.1427, 1.2046),
            (2.8366, -3.0525, 1.2012),
        ],
        "cycle",
    ),
    "polar_express": (
        [
            (8.2051, -22.9019, 16.4607),
            (4.0664, -2.8612, 0.5184),
            (3.9096, -2.8234, 0.5250),
            (3.2856, -2.4153, 0.4853),
            (2.2779, -1.6198, 0.3985),
            (1.8726, -1.2307, 0.3585),
            (1.8564, -1.2132, 0.3568),
            (1.8750, -1.2500, 0.3750),
        ],
        "repeat_last",
    ),
    "cubic5": (
        [
            (3.3656576, -3.3420992, 0.0),
            (2.5744352, -1.4957376, 0.0),
            (2.5368962, -1.4312570, 0.0),
            (2.4418906, -1.2764040, 0.0),
            (2.2230472, -0.9630650, 0.0),
        ],
        "cycle",
    ),
}


def schedule(kind, steps):
    table, mode = TABLES[kind]
    n = len(table)
    return [table[i % n] if mode == "cycle" else table[min(i, n - 1)] for i in range(steps)]


def main():
    rng = random.Random(20251125)
    cases = []
    for rows, cols, kind, steps in [
        (8, 16, "simple", 5),
        (16, 8, "quintic", 5),
        (16, 16, "polar_express", 10),
        (8, 24, "cubic5", 5),
        (32, 16, "simple", 3),
        (16, 32, "quintic", 7),
    ]:
        r = min(rows, cols)
        # powers of two: exactly representable in bf16 and float32
        s = [2.0 ** rng.randint(-6, 0) * rng.choice((-1.0, 1.0)) for _ in range(r)]
        row_of = rng.sample(range(rows), r)
        col_of = rng.sample(range(cols), r)
        norm = math.sqrt(sum(v * v for v in s))
        t = [v / norm for v in s]
        for a, b, c in schedule(kind, steps):
            t = [a * v + b * v**3 + c * v**5 for v in t]
        cases.append(
            dict(rows=rows, cols=cols, coefficient_type=kind, steps=steps, row_of=row_of, col_of=col_of, values=s, expected=t)
        )
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    with open(out, "w") as f:
        json.dump(dict(description="x[row_of[i], col_of[i]] = values[i]; result[row_of[i], col_of[i]] = expected[i]; zeros elsewhere", cases=cases), f, indent=1)
    print("wrote", out, len(cases), "cases")


if __name__ == "__main__":
    main()

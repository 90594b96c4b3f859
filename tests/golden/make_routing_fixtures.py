"""Writes tests/golden/routing_cases.json: tiny routing / capacity cases whose
expected outputs come from the pure-Python sequential loops of oracle/routing.py
(small enough to follow by hand).  The reference ships no golden vectors for
this path (its tests compare against a brute-force model built in-process), so
these are the fixtures the C oracle and the HIP kernels are both held to.

Run from the repository root:  python tests/golden/make_routing_fixtures.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import routing  # noqa: E402


def case(name, gate, n_expert, cap):
    gate = [int(g) for g in gate]
    counts = [sum(1 for g in gate if g == e) for e in range(n_expert)]
    pos, cum_after = routing.assign_pos_py(counts, gate)
    pruned, cap_after = routing.prune_py(gate, [min(c, cap) for c in counts])
    return {"name": name, "n_expert": n_expert, "gate": gate, "counts": counts, "pos": pos,
            "cum_after": cum_after, "capacity": cap, "limited": [min(c, cap) for c in counts],
            "pruned": pruned, "cap_after": cap_after}


def main():
    rng = np.random.default_rng(20240229)
    cases = [
        case("hand_top2", [1, 0, 0, 1, 1, 2, 0, 1], 3, 2),
        case("with_drops", [2, -1, 0, 2, -1, 2, 1, 0, 2, -1], 4, 1),
        case("single_expert", [0] * 7, 1, 3),
        case("all_dropped", [-1] * 5, 2, 1),
        case("empty", [], 3, 1),
        case("one_slot", [4], 6, 0),
    ]
    for n, e in ((70, 5), (130, 16), (300, 3), (2100, 9)):
        g = rng.integers(-1, e, size=n)
        cases.append(case(f"random_{n}_{e}", g, e, max(1, n // (2 * e))))
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "routing_cases.json")
    with open(out, "w") as f:
        json.dump(cases, f, separators=(",", ":"))
    print(out, len(cases))


if __name__ == "__main__":
    main()

"""Writes cg_tables_sympy.json: exact Clebsch-Gordan tables from sympy radicals, printed to 17 digits.

Covers every triple with l1,l2 <= 4, the triples named by the benchmark configurations ((2,3,4), L<=6 diagonal
is covered through l1,l2<=6 for l<=6 on a sparse subset) and three l1=l2=10 tables (l=0,7,20).
Run:  python tests/golden/make_cg_tables.py      (about a minute)
"""
import json
import os

from sympy import S
from sympy.physics.quantum.cg import CG


def table(l1, l2, l):
    rows = []
    for m1 in range(-l1, l1 + 1):
        row = []
        for m2 in range(-l2, l2 + 1):
            if abs(m1 + m2) <= l:
                row.append(float(CG(S(l1), S(m1), S(l2), S(m2), S(l), S(m1 + m2)).doit().evalf(30)))
            else:
                row.append(0.0)
        rows.append(row)
    return rows


def main():
    todo = set()
    for l1 in range(5):
        for l2 in range(5):
            for l in range(abs(l1 - l2), l1 + l2 + 1):
                todo.add((l1, l2, l))
    todo |= {(5, 5, 0), (5, 6, 3), (6, 6, 6), (6, 5, 2), (6, 6, 12), (6, 3, 4), (10, 10, 0), (10, 10, 7), (10, 10, 20)}
    out = {}
    for t in sorted(todo):
        out["%d,%d,%d" % t] = table(*t)
        print(t, flush=True)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cg_tables_sympy.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

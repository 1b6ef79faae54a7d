"""Writes tests/golden/glu_kat.json: known answers for the clamped SwiGLU of the GPT-OSS expert MLP,
    h = (clamp(U, -7, 7) + 1) * g * sigmoid(1.702 * g),  g = min(G, 7),
computed in double precision with Python's math module only (no torch, no oracle code), so that the
fixture is independent of everything it checks.  The definition is the one in drbh/yamoe
(csrc/moe.cpp:164-180; reference.py:49-54).  Run from the repo root: python tests/golden/make_glu_kat.py
"""
import json
import math
import os


def h(G, U):
    g = min(G, 7.0)
    u = max(-7.0, min(7.0, U))
    s = 1.0 / (1.0 + math.exp(-1.702 * g))
    return (u + 1.0) * g * s


CASES = [(0.0, 3.0), (1.0, 0.0), (1.0, -1.0), (-1.0, 2.0), (7.0, 7.0), (100.0, 100.0), (100.0, -100.0),
         (-50.0, 5.0), (6.999, -6.999), (7.001, 7.001), (0.5, 0.25), (-3.25, -0.75), (2.0, 1.5)]

if __name__ == "__main__":
    out = [dict(G=G, U=U, h=h(G, U)) for G, U in CASES]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "glu_kat.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)

"""Writes tests/golden/notebook_blocks.json: known answers for the reference's notebook walkthrough
(MeshFlowCPU.ipynb cells 2-4: 4x2 mesh, (B,I,O)=(512,256,1024), X=arange/(B*I), W=arange/(I*O),
dY=1/(B*O)).

The reference stores no outputs and JAX is not installed, so the answers come from exact integer
arithmetic: every operand is an integer over a power of two, hence every entry of X@W, dY@W^T and
X^T@dY is an exact rational that float64 represents without rounding.  Per mesh device the file holds
the sum, the sum of squares and the four corner values of that device's output block.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
from fractions import Fraction

Bt, I, O = 512, 256, 1024
R, C = 4, 2


def y(r, c):      # (X @ W)[r, c]
    s1 = I * (I - 1) // 2
    s2 = (I - 1) * I * (2 * I - 1) // 6
    return Fraction(r * I * O * s1 + r * I * c * I + O * s2 + c * s1, (Bt * I) * (I * O))


def dx(r, i):     # (dY @ W^T)[r, i]
    return Fraction(i * O * O + O * (O - 1) // 2, (I * O) * (Bt * O))


def dw(i, o):     # (X^T @ dY)[i, o]
    return Fraction(I * Bt * (Bt - 1) // 2 + Bt * i, (Bt * I) * (Bt * O))


def block_stats(f, rows, cols):
    out = {}
    for bi in range(R):
        for bj in range(C):
            r0, r1 = bi * rows // R, (bi + 1) * rows // R
            c0, c1 = bj * cols // C, (bj + 1) * cols // C
            tot = Fraction(0); sq = Fraction(0)
            for r in range(r0, r1):
                for c in range(c0, c1):
                    v = f(r, c); tot += v; sq += v * v
            out[f"{bi},{bj}"] = {
                "sum": float(tot), "sumsq": float(sq),
                "corners": [float(f(r0, c0)), float(f(r0, c1 - 1)), float(f(r1 - 1, c0)), float(f(r1 - 1, c1 - 1))],
            }
    return out


def main():
    data = {
        "mesh": [R, C], "B": Bt, "I": I, "O": O, "K": 8, "blocksize": 8,
        "os": block_stats(y, Bt, O),      # Y  = OS(X, W)   [512, 1024]
        "ls": block_stats(dx, Bt, I),     # dX = LS(dY, W)  [512, 256]
        "rs": block_stats(dw, I, O),      # dW = RS(X, dY)  [256, 1024]
    }
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "notebook_blocks.json"), "w") as f:
        json.dump(data, f, indent=1)


if __name__ == "__main__":
    main()

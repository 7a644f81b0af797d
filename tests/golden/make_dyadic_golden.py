"""Writes tests/golden/dyadic_4x4.json: known-answer vectors for IF / LIF / PLIF forward.

Input: the one literal input of the reference's test-suite
(test/activation_based/test_triton_neuron.py:1207-1216): a 4x4 matrix of dyadic rationals,
v_init = 0, 1/tau = 0.5, v_threshold = 1, v_reset in {0, None}.  The expected spikes, h and v
are computed here with exact rational arithmetic (``fractions.Fraction``) from the definitions
  IF    h = v + x
  LIF   h = v + (x - (v - vr))/tau          (decay_input)      h = v - (v - vr)/tau + x   (otherwise)
  fire  s = [h >= v_th]
  reset hard v = s*vr + (1-s)*h             soft v = h - s*v_th
and every value is checked to be exactly representable in bf16 (hence fp16 and fp32), so any IEEE
implementation in any op order must reproduce them bit for bit.  Each case scales the input by
``scale`` (1 = the reference's input; 4 = a second family in which LIF/PLIF fire as well).
No reference code is run.
"""

import json
import os
from fractions import Fraction as Fr

X = [
    ["1/4", "1/2", "3/4", "1"],
    ["1/2", "-1/4", "1/4", "-1/2"],
    ["1/4", "3/4", "-1/2", "1/2"],
    ["-1/4", "1/2", "1/4", "3/4"],
]


def representable(fr: Fr, mant_bits: int) -> bool:
    if fr == 0:
        return True
    num, den = abs(fr.numerator), fr.denominator
    if den & (den - 1):
        return False
    while num % 2 == 0:
        num //= 2
    return num.bit_length() <= mant_bits


def run(kind, decay_input, v_reset, k=Fr(1, 2), v_th=Fr(1), scale=1):
    x = [[Fr(e) * scale for e in row] for row in X]
    T, N = len(x), len(x[0])
    vr = Fr(0) if v_reset is None else Fr(v_reset)
    v = [Fr(0)] * N
    S, H, V = [], [], []
    for t in range(T):
        s_row, h_row, v_row = [], [], []
        for n in range(N):
            if kind == "if":
                h = v[n] + x[t][n]
            elif decay_input:
                h = v[n] + (x[t][n] - (v[n] - vr)) * k
            else:
                h = v[n] - (v[n] - vr) * k + x[t][n]
            s = 1 if h >= v_th else 0
            vn = (h - s * v_th) if v_reset is None else (s * vr + (1 - s) * h)
            for val in (h, vn):
                assert representable(val, 8), (kind, t, n, val)  # fits bf16, hence fp16 and fp32
            s_row.append(s)
            h_row.append(float(h))
            v_row.append(float(vn))
            v[n] = vn
        S.append(s_row)
        H.append(h_row)
        V.append(v_row)
    return {"spike": S, "h": H, "v": V}


def main():
    cases = []
    for kind in ("if", "lif", "plif"):
        for v_reset in (0.0, None):
            for decay_input in ((True,) if kind == "if" else (True, False)):
                out = run(kind, decay_input, v_reset)
                cases.append({"kind": kind, "v_reset": v_reset, "decay_input": decay_input, "k": 0.5,
                              "v_threshold": 1.0, **out})
    # second family (not from the reference): the same matrix times 4 so that LIF/PLIF fire too, with a
    # dyadic negative reset value added; still exact in bf16/fp16/fp32.
    for kind in ("if", "lif", "plif"):
        for v_reset in (0.0, -0.25, None):
            for decay_input in ((True,) if kind == "if" else (True, False)):
                out = run(kind, decay_input, v_reset, scale=4)
                cases.append({"kind": kind, "v_reset": v_reset, "decay_input": decay_input, "k": 0.5,
                              "v_threshold": 1.0, "scale": 4.0, **out})
    for c in cases:
        c.setdefault("scale", 1.0)
    doc = {"x": [[float(Fr(e)) for e in row] for row in X], "v_init": [0.0] * 4, "cases": cases}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dyadic_4x4.json")
    with open(path, "w") as f:
        json.dump(doc, f, indent=1)
    print("wrote", path, len(cases), "cases")


if __name__ == "__main__":
    main()

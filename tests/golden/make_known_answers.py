"""Writes tests/golden/lce_known_answers.json: closed-form values of log-prob and entropy for logit
vectors whose softmax can be written down exactly, evaluated with mpmath at 40 digits.  Nothing of the
reference is imported or run; the first family is the construction of the reference's padded-vocabulary
regression test (tests/utils/test_linear_cross_entropy.py:352-395: one logit +3, V-1 logits -15, label 0).

    python tests/golden/make_known_answers.py
"""

import json
import os

import mpmath as mp

mp.mp.dps = 40


def two_level(z0, z1, n1):
    """One logit z0 (the label) and n1 logits z1."""
    z0, z1 = mp.mpf(z0), mp.mpf(z1)
    lse = z0 + mp.log1p(n1 * mp.exp(z1 - z0))
    p0, p1 = mp.exp(z0 - lse), mp.exp(z1 - lse)
    return z0 - lse, lse - (p0 * z0 + n1 * p1 * z1)


def main():
    out = {"two_level": [], "uniform": []}
    for V in (152064, 149 * 1024, 151936, 128256):
        lp, ent = two_level(3, -15, V - 1)
        out["two_level"].append({"V": V, "z0": 3.0, "z1": -15.0, "logprob": mp.nstr(lp, 30), "entropy": mp.nstr(ent, 30)})
    for z0, z1, V in ((0.5, -0.25, 11), (10, 0, 256), (-2, 1, 4099)):
        lp, ent = two_level(z0, z1, V - 1)
        out["two_level"].append({"V": V, "z0": float(z0), "z1": float(z1), "logprob": mp.nstr(lp, 30), "entropy": mp.nstr(ent, 30)})
    for V in (2, 11, 256, 4099, 128256, 151936, 152064):
        out["uniform"].append({"V": V, "logprob": mp.nstr(-mp.log(V), 30), "entropy": mp.nstr(mp.log(V), 30)})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lce_known_answers.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    main()

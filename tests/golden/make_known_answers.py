"""Writes tests/golden/lce_known_answers.json: closed-form values of log-prob and entropy for logit
vectors whose softmax can be written down exactly, evaluated with mpmath at 40 digits.  Nothing of the
reference is imported or run; the first family is the construction of the reference's padded-vocabulary
regression test (tests/utils/test_linear_cross_entropy.py:352-395: one logit +3, V-1 logits -15, label 0).
The "ppo" family evaluates the formulas of the clipped policy loss, the KL estimators and the aggregation modes
(verl/trainer/ppo/core_algos.py:1172-1204, :1336-1369, :2228-2245) on a 3 x 4 batch with plain scalar arithmetic.

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


def ppo_case():
    """A 3 x 4 batch that visits every branch: ratio inside the clip range, clipped above and below, dual clip
    (A < 0 and ratio > 3), the +-20 clamp of the log-ratio, a masked-out token with a huge value, a fully masked row."""
    f = mp.mpf
    lp = [[f("-1.0"), f("-0.5"), f("-2.0"), f("-0.25")], [f("-1.5"), f("-0.75"), f("-3.0"), f("-0.125")], [f("-1.0")] * 4]
    old = [[f("-1.0625"), f("-0.25"), f("-3.5"), f("-25.0")], [f("-1.25"), f("-2.0"), f("-2.875"), f("1000.0")], [f("-1.0")] * 4]
    ref = [[f("-1.25"), f("-0.5"), f("-1.0"), f("-0.3125")], [f("-1.0"), f("-0.875"), f("-30.0"), f("0.0")], [f("-2.0")] * 4]
    adv = [[f("1.5")] * 4, [f("-0.75")] * 4, [f("2.0")] * 4]
    ent = [[f("0.5"), f("1.25"), f("2.0"), f("0.125")], [f("3.0"), f("0.25"), f("1.0"), f("7.0")], [f("1.0")] * 4]
    mask = [[1, 1, 1, 1], [1, 1, 1, 0], [0, 0, 0, 0]]
    lo, hi, c = f("0.2"), f("0.3"), f("3.0")
    clamp = lambda x, a, b: max(a, min(b, x))
    loss, kls = [], {k: [] for k in ("kl", "abs", "mse", "low_var_kl")}
    clipped = lower = nkl_sum = f(0)
    for i in range(3):
        loss.append([])
        for k in kls:
            kls[k].append([])
        for j in range(4):
            nkl = clamp(lp[i][j] - old[i][j], f(-20), f(20))
            r = mp.exp(nkl)
            l1, l2, l3 = -adv[i][j] * r, -adv[i][j] * clamp(r, 1 - lo, 1 + hi), -adv[i][j] * c
            lc1 = max(l1, l2)
            loss[i].append(min(l3, lc1) if adv[i][j] < 0 else lc1)
            if mask[i][j]:
                clipped += 1 if l2 > l1 else 0
                lower += 1 if (lc1 > l3 and adv[i][j] < 0) else 0
                nkl_sum += -nkl
            d = lp[i][j] - ref[i][j]
            q = clamp(-d, f(-20), f(20))
            kls["kl"][i].append(d)
            kls["abs"][i].append(abs(d))
            kls["mse"][i].append(d * d / 2)
            kls["low_var_kl"][i].append(clamp(mp.exp(q) - q - 1, f(-10), f(10)))
    ntok = sum(map(sum, mask))

    def agg(mat, mode):
        rows = [sum(mat[i][j] * mask[i][j] for j in range(4)) for i in range(3)]
        cnt = [sum(mask[i]) for i in range(3)]
        live = [i for i in range(3) if cnt[i] > 0]
        if mode == "token-mean":
            return sum(rows) / ntok
        if mode == "token-sum":
            return sum(rows)
        if mode == "seq-mean-token-sum":
            return sum(rows[i] for i in live) / len(live)
        if mode == "seq-mean-token-sum-norm":
            return sum(rows[i] for i in live) / len(live) / 4
        return sum(rows[i] / (cnt[i] + f("1e-8")) for i in live) / len(live)

    modes = ("token-mean", "token-sum", "seq-mean-token-sum", "seq-mean-token-sum-norm", "seq-mean-token-mean")
    s = lambda x: mp.nstr(x, 30)
    flat = lambda m: [[float(v) for v in row] for row in m]
    return {
        "log_prob": flat(lp), "old_log_prob": flat(old), "ref_log_prob": flat(ref), "advantages": flat(adv), "entropy": flat(ent),
        "mask": mask, "clip_ratio_low": 0.2, "clip_ratio_high": 0.3, "clip_ratio_c": 3.0,
        "pg_losses": [[s(v) for v in row] for row in loss],
        "kl": {k: [[s(v) for v in row] for row in m] for k, m in kls.items()},
        "pg_loss": {m: s(agg(loss, m)) for m in modes},
        "entropy_loss": {m: s(agg(ent, m)) for m in modes},
        "kl_loss": {k: {m: s(agg(kls[k], m)) for m in modes} for k in kls},
        # the three metrics are masked means, sum / (count + 1e-8) (verl/utils/torch_functional.py:294-308)
        "pg_clipfrac": s(clipped / (ntok + f("1e-8"))), "pg_clipfrac_lower": s(lower / (ntok + f("1e-8"))),
        "ppo_kl": s(nkl_sum / (ntok + f("1e-8"))),
    }


def main():
    out = {"two_level": [], "uniform": [], "ppo": ppo_case()}
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

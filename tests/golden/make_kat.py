"""Re-derives the known-answer vectors in kat.json with exact Python integer arithmetic.

Independent of the oracle and of the product: only the formulas cited in README.md.
Run:  python tests/golden/make_kat.py
"""
import json
import os
from fractions import Fraction


def act(acc, bias, scale, shift, zp, lo, hi):
    """ACT rescale-clamp with exact rationals: floor(x / 2^shift + 1/2) is round-half-up."""
    t1 = (acc + bias) * scale
    t3 = (Fraction(t1, 1 << shift) + Fraction(1, 2)).__floor__() if shift > 0 else t1
    return max(lo, min(hi, t3 + zp))


def trunc(x):
    return int(x)  # C cast of a double: toward zero


def add_case():
    # input 0: rescale(2^30, 10, zp -2) then rescale(1515257681, 32); input 1: rescale(2^30, 11, zp -3)
    # output: rescale(1093202297, 49, out zp -2)
    in0 = (2 ** 30 / 2 ** 10) * (1515257681 / 2 ** 32)
    in1 = 2 ** 30 / 2 ** 11
    out = 1093202297 / 2 ** 49
    m0, m1 = out * in0, out * in1
    S = 1 << 12
    w0, w1 = trunc(m0 * S), trunc(m1 * S)
    bias = -trunc(m0 * S * -2) - trunc(m1 * S * -3)
    pairs = [(0, 0), (10, -20), (127, 127), (-128, -128), (-2, -3), (5, 7), (-77, 33), (100, -100)]
    return {
        "source": "tests/testdata/tosa_ops/add.mlir:3-23",
        "m0": m0, "m1": m1, "zp0": -2, "zp1": -3,
        "weights": [w0, w1], "scale_bias": [bias, 1], "shift_factor": 12, "output_zp": -2,
        "output_min": -128, "output_max": 127,
        "inputs": pairs,
        "expected": [act(a * w0 + b * w1, bias, 1, 12, -2, -128, 127) for a, b in pairs],
    }


def fc_case():
    w_kf = [[1, 2], [3, 4], [5, 6]]              # [K, F] as in the fixture
    w_fk = [[w_kf[k][f] for k in range(3)] for f in range(2)]  # TorqHL [F, K]
    bias = [7, -9]
    xs = [[1, 1, 1], [-40, 0, 40], [-1, -1, -1], [127, 127, 127], [-128, -128, -128], [3, -2, 1]]
    exp = []
    for x in xs:
        exp.append([act(sum(a * b for a, b in zip(x, w_fk[f])), bias[f], 1 << 30, 30, 3, -128, 127)
                    for f in range(2)])
    return {
        "source": "tests/testdata/linalg_ops/conv1d-matmul-fc-i8-bias-requant.mlir:23-26,73-78",
        "weights_fk": w_fk, "multiplier": [1 << 30, 1 << 30], "shift": [30, 30], "tosa_bias": bias,
        "scale_bias": [7, 1 << 30, -9, 1 << 30], "shift_factor": 30, "output_zp": 3,
        "output_min": -128, "output_max": 127, "inputs": xs, "expected": exp,
    }


def avgpool_case():
    H = W = 7
    in_zp, out_zp = 4, 0
    scale = (1 << 20) // (H * W)
    bias = -(H * W * in_zp)
    vals = [4, 5, 127, -128, 0, -1, 64]
    return {
        "source": "tests/testdata/tosa_ops/avgpool2d.mlir:3-4 (7x7x128, in zp 4, out zp 0)",
        "H": H, "W": W, "input_zp": in_zp, "output_zp": out_zp, "scale_bias": [bias, scale],
        "shift_factor": 20, "output_min": -128, "output_max": 127,
        "constant_inputs": vals,
        "expected": [act(H * W * v, bias, scale, 20, out_zp, -128, 127) for v in vals],
    }


def requant_ties():
    # t1 = k * 2^sh + 2^(sh-1): exactly half way; NTP rounds toward +inf.
    cases = []
    for sh in (1, 4, 12, 31, 40):
        for k in (-3, -1, 0, 2):
            # acc chosen so that acc * scale is the tie: scale = 2^(sh-1), acc = 2k + 1
            scale = 1 << (sh - 1) if sh - 1 < 31 else None
            if scale is None:
                continue
            acc = 2 * k + 1
            cases.append({"acc": acc, "bias": 0, "scale": scale, "shift": sh, "zp": 0,
                          "min": -(1 << 31), "max": (1 << 31) - 1, "expected": k + 1})
    return cases


def main():
    kat = {"add_tosa_add_mlir": add_case(), "fc_conv1d_matmul_fc_requant": fc_case(),
           "avgpool_7x7": avgpool_case(), "requant_ties": requant_ties()}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat.json")
    with open(path, "w") as f:
        json.dump(kat, f, indent=1)
        f.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    main()

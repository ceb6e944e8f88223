"""Writes tests/golden/hand_cases.json: tiny cases worked out with plain Python arithmetic
(no torch, no numpy, none of this repository's code), small enough to verify by hand.

The reference repository holds no golden vectors, fixtures or tests for this path, and its
kernels cannot run without a GPU and Triton, so these are the only committed vectors; they
pin the conventions a plausible mistake would break (expert-major / token-ascending order,
slot numbering, first-half-linear / second-half-SiLU split of Wl1, gate weight applied
after the down projection, renormalised top-k weights).

Usage: python tests/golden/make_hand_cases.py
"""
import json
import math
import os


def index_case():
    # 4 experts x 6 tokens, every token held by exactly 2 experts
    mask = [[1, 0, 1, 0, 0, 1],
            [0, 1, 1, 0, 1, 0],
            [0, 0, 0, 1, 0, 0],
            [1, 1, 0, 1, 1, 1]]
    N, M = len(mask), len(mask[0])
    sizes = [sum(row) for row in mask]
    cumsums = [0]
    for v in sizes:
        cumsums.append(cumsums[-1] + v)
    idx, which = [], []
    for i in range(N):
        for m in range(M):
            if mask[i][m]:
                idx.append(m)
                which.append(sum(mask[j][m] for j in range(i)))  # lower-numbered experts holding m
    K = 2
    inv = [[None] * K for _ in range(M)]
    for r, (m, k) in enumerate(zip(idx, which)):
        inv[m][k] = r
    return {"mask_NM": mask, "K": K, "sizes_N": sizes, "cumsums_N": cumsums, "idx_Msum": idx,
            "which_Msum": which, "inv_MK": inv}


def experts_case():
    # M=2 tokens, D=2, H=1, N=2 experts, K=1: token 0 -> expert 1, token 1 -> expert 0.
    # Wl1[i] is [D, 2H]: column 0 = linear half a, column 1 = SiLU half b.
    x = [[1.0, 2.0], [0.5, -1.0]]
    Wl1 = [[[1.0, 0.5], [0.0, 0.25]],     # expert 0
           [[2.0, -1.0], [1.0, 0.5]]]     # expert 1
    Wl2 = [[[1.0, -2.0]],                 # expert 0: [H, D]
           [[0.5, 4.0]]]                  # expert 1
    mask = [[0, 1], [1, 0]]
    s = [[0.0, 0.25], [0.5, 0.0]]
    y = []
    for m, e, sv in ((0, 1, 0.5), (1, 0, 0.25)):
        a = x[m][0] * Wl1[e][0][0] + x[m][1] * Wl1[e][1][0]
        b = x[m][0] * Wl1[e][0][1] + x[m][1] * Wl1[e][1][1]
        h = a * b / (1.0 + math.exp(-b))
        y.append([sv * h * Wl2[e][0][0], sv * h * Wl2[e][0][1]])
    # token 0: a = 1*2 + 2*1 = 4, b = 1*(-1) + 2*0.5 = 0 -> h = 0 -> y = [0, 0]
    # token 1: a = 0.5, b = 0.25 - 0.25 = 0 -> h = 0 as well; so use a second pair with b != 0
    x2 = [[1.0, 1.0], [2.0, 0.0]]
    y2 = []
    for m, e, sv in ((0, 1, 0.5), (1, 0, 0.25)):
        a = x2[m][0] * Wl1[e][0][0] + x2[m][1] * Wl1[e][1][0]
        b = x2[m][0] * Wl1[e][0][1] + x2[m][1] * Wl1[e][1][1]
        h = a * b / (1.0 + math.exp(-b))
        y2.append([sv * h * Wl2[e][0][0], sv * h * Wl2[e][0][1]])
    # token 0 (expert 1): a = 3, b = -0.5, h = 3*(-0.5)*sigmoid(-0.5) = -0.566311...
    # token 1 (expert 0): a = 2, b = 1,    h = 2*sigmoid(1)         =  1.462117...
    return {"Wl1_ND2H": Wl1, "Wl2_NHD": Wl2, "mask_NM": mask, "s_NM": s,
            "x_zero_gate": x, "y_zero_gate": y, "x": x2, "y": y2}


def router_case():
    # 2 tokens, 4 routed experts, K=2, no shared experts, zero bias
    logits = [[0.0, math.log(2.0), math.log(4.0), math.log(1.0)],
              [math.log(3.0), 0.0, 0.0, math.log(3.0)]]
    mask_MN, s_MN = [], []
    for row in logits:
        e = [math.exp(v) for v in row]
        p = [v / sum(e) for v in e]
        order = sorted(range(4), key=lambda i: (-p[i], i))[:2]  # ties -> lower index
        tot = sum(p[i] for i in order)
        mask_MN.append([1 if i in order else 0 for i in range(4)])
        s_MN.append([p[i] / tot if i in order else 0.0 for i in range(4)])
    # token 0: p = [1,2,4,1]/8 -> experts 2 and 1, weights 2/3 and 1/3
    # token 1: p = [3,1,1,3]/8 -> experts 0 and 3, weights 1/2 and 1/2
    return {"logits_MN": logits, "K": 2, "Ks": 0, "mask_MN": mask_MN, "s_MN": s_MN}


if __name__ == "__main__":
    out = {"index": index_case(), "experts": experts_case(), "router": router_case()}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hand_cases.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)

"""Writes tests/golden/adder_small_int.json: tiny integer-valued AdderNet layers with exact answers.

The reference ships no golden vectors (its only check, adder_cuda/test_cuda.py,
prints statistics of random cases), so these are produced here by literal
integer loop nests over the definitions the reference states
(adder_cuda/test_cuda.py:18-22, 35-41, 57-60 through the im2col of adder.py:26-34):

    y[n,co,ho,wo]   = -sum |w[co,ci,i,j] - xpad[n,ci,ho*s+i-p,wo*s+j-p]|
    gw[co,ci,i,j]   =  sum (xpad - w) * gy
    gx[n,ci,hi,wi]  =  sum clamp(w - x, -1, 1) * gy      (padding taps dropped)

Inputs are small integers, so every value is exact in fp32 and can be checked by
hand.  Run from the repository root:  python tests/golden/make_fixtures.py
"""
import json
import os
import random

CASES = [  # N, Ci, H, W, Co, k, stride, pad
    (2, 3, 5, 5, 4, 3, 1, 1),
    (2, 3, 5, 5, 4, 3, 2, 1),
    (2, 3, 5, 5, 4, 3, 1, 0),
    (2, 3, 6, 5, 4, 1, 2, 0),
    (1, 2, 4, 6, 3, 3, 2, 1),
    # large enough for the tiled GPU kernels (>= 8 channels): stride 1, stride 2, and a layer with more than
    # 2304 terms per input position (a different arithmetic form of the input gradient on the GPU)
    (2, 8, 8, 8, 8, 3, 1, 1),
    (2, 8, 8, 8, 16, 3, 2, 1),
    (1, 8, 4, 4, 260, 3, 1, 1),
    (2, 64, 4, 4, 64, 1, 1, 0),
]


def clamp(v):
    return -1 if v < -1 else (1 if v > 1 else v)


def solve(N, Ci, H, W, Co, k, s, p, rng):
    Ho, Wo = (H - k + 2 * p) // s + 1, (W - k + 2 * p) // s + 1
    x = [[[[rng.randint(-3, 3) for _ in range(W)] for _ in range(H)] for _ in range(Ci)] for _ in range(N)]
    w = [[[[rng.randint(-3, 3) for _ in range(k)] for _ in range(k)] for _ in range(Ci)] for _ in range(Co)]
    gy = [[[[rng.randint(-2, 2) for _ in range(Wo)] for _ in range(Ho)] for _ in range(Co)] for _ in range(N)]
    y = [[[[0] * Wo for _ in range(Ho)] for _ in range(Co)] for _ in range(N)]
    gw = [[[[0] * k for _ in range(k)] for _ in range(Ci)] for _ in range(Co)]
    gx = [[[[0] * W for _ in range(H)] for _ in range(Ci)] for _ in range(N)]
    for n in range(N):
        for co in range(Co):
            for ho in range(Ho):
                for wo in range(Wo):
                    g = gy[n][co][ho][wo]
                    for ci in range(Ci):
                        for i in range(k):
                            for j in range(k):
                                hi, wi = ho * s + i - p, wo * s + j - p
                                inside = 0 <= hi < H and 0 <= wi < W
                                xv = x[n][ci][hi][wi] if inside else 0
                                wv = w[co][ci][i][j]
                                y[n][co][ho][wo] -= abs(wv - xv)
                                gw[co][ci][i][j] += (xv - wv) * g
                                if inside:
                                    gx[n][ci][hi][wi] += clamp(wv - xv) * g
    return {"dims": [N, Ci, H, W, Co, k, s, p], "x": x, "w": w, "gy": gy, "y": y, "gw": gw, "gx": gx}


def main():
    rng = random.Random(20240531)
    out = [solve(*c, rng) for c in CASES]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "adder_small_int.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

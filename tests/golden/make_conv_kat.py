"""Writes tests/golden/conv_kat.json: known-answer convolutions / linear layers by plain Python loops.

Operands are multiples of 1/8 with small magnitude, so every partial sum is exactly representable in float32 and the
expected outputs are exact whatever the summation order: any implementation (oracle, C restatement, HIP kernel with
bf16 operands - multiples of 1/8 below 32 are exact in bf16 too) must reproduce them bit for bit.
Layouts as in torch.nn.functional.conv2d: x [N, Cin, H, W], w [Cout, Cin/groups, KH, KW], out [N, Cout, Ho, Wo].

Run from the repository root:  python tests/golden/make_conv_kat.py
"""
import json
import os
import random


def conv2d(x, w, b, N, Cin, H, W, Cout, KH, KW, sh, sw, ph, pw, groups):
    Ho = (H + 2 * ph - KH) // sh + 1
    Wo = (W + 2 * pw - KW) // sw + 1
    cg, og = Cin // groups, Cout // groups
    out = []
    for n in range(N):
        for oc in range(Cout):
            g = oc // og
            for oh in range(Ho):
                for ow in range(Wo):
                    acc = b[oc]
                    for ci in range(cg):
                        for kh in range(KH):
                            ih = oh * sh - ph + kh
                            if not 0 <= ih < H:
                                continue
                            for kw in range(KW):
                                iw = ow * sw - pw + kw
                                if not 0 <= iw < W:
                                    continue
                                acc += x[((n * Cin + g * cg + ci) * H + ih) * W + iw] * w[((oc * cg + ci) * KH + kh) * KW + kw]
                    out.append(acc)
    return out, Ho, Wo


def main():
    rnd = random.Random(7)
    grid = lambda count, lo, hi: [rnd.randint(lo, hi) / 8.0 for _ in range(count)]
    cases = []
    configs = [
        # N Cin H  W  Cout KH KW sh sw ph pw groups
        (1, 2, 5, 5, 3, 3, 3, 1, 1, 1, 1, 1),
        (2, 3, 6, 7, 4, 3, 3, 2, 2, 1, 1, 1),
        (1, 4, 4, 4, 5, 1, 1, 1, 1, 0, 0, 1),
        (1, 2, 7, 7, 2, 5, 5, 1, 1, 2, 2, 1),
        (1, 3, 9, 9, 2, 7, 7, 2, 2, 3, 3, 1),
        (1, 1, 15, 15, 2, 11, 11, 4, 4, 2, 2, 1),
        (2, 4, 5, 6, 4, 3, 3, 1, 1, 1, 1, 4),
        (1, 4, 6, 6, 4, 3, 3, 2, 2, 1, 1, 4),
    ]
    for (N, Cin, H, W, Cout, KH, KW, sh, sw, ph, pw, groups) in configs:
        x = grid(N * Cin * H * W, -8, 8)
        w = grid(Cout * (Cin // groups) * KH * KW, -4, 4)
        b = grid(Cout, -8, 8)
        out, Ho, Wo = conv2d(x, w, b, N, Cin, H, W, Cout, KH, KW, sh, sw, ph, pw, groups)
        cases.append({"kind": "conv2d", "N": N, "Cin": Cin, "H": H, "W": W, "Cout": Cout, "KH": KH, "KW": KW,
                      "stride": [sh, sw], "padding": [ph, pw], "groups": groups, "Ho": Ho, "Wo": Wo,
                      "x": x, "w": w, "b": b, "out": out})
    for (M, Fin, Fout) in [(3, 8, 5), (1, 40, 17), (5, 33, 16)]:
        x = grid(M * Fin, -8, 8)
        w = grid(Fout * Fin, -4, 4)
        b = grid(Fout, -8, 8)
        out = [b[o] + sum(x[m * Fin + k] * w[o * Fin + k] for k in range(Fin)) for m in range(M) for o in range(Fout)]
        cases.append({"kind": "linear", "M": M, "Fin": Fin, "Fout": Fout, "x": x, "w": w, "b": b, "out": out})
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "conv_kat.json")
    with open(path, "w") as fh:
        json.dump({"cases": cases}, fh)
    print(f"wrote {len(cases)} cases to {path}")


if __name__ == "__main__":
    main()

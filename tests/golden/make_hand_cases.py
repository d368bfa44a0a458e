"""Writes tests/golden/reference_hand_cases.json.

Inputs are the literal arrays of the reference's own convolution tests (pydtnn/tests/conv_gemm.py:81-84,
101-106, 123-134, 151-155, 172-180, 197-209 and pydtnn/tests/conv2d_conv_gemm.py:72-103); those tests store no
expected outputs (they compare two code paths), so the expected y here is the defining sum
    y[n, co, oy, ox] = sum_{c,i,j} w[co,c,i,j] * x[n, c, sv*oy + dv*i - pv, sh*ox + dj*j - ph]
evaluated with Python integers (every value is a small integer, so the result is exact in fp32 too).
Nothing of the build is imported.  Run:  python tests/golden/make_hand_cases.py
"""
import json
import os

x_2x4 = [[[[1, 2, 4, 8], [16, 32, 64, 128]]]]
x_2x4_c2 = [[[[1, 2, 4, 8], [16, 32, 64, 128]], [[128, 256, 512, 1024], [2048, 4096, 8192, 16384]]]]
x_4x4 = [[[[1, 2, 4, 8], [16, 32, 64, 128], [1, 2, 4, 8], [16, 32, 64, 128]]]]
x_4x8 = [[[[1, 2, 4, 8, 9, 10, 11, 12], [16, 32, 64, 128, 129, 130, 131, 132],
           [1, 2, 4, 8, 9, 10, 11, 12], [16, 32, 64, 128, 129, 130, 131, 132]]]]
x_8x8 = [[[[c + 10 * r for c in range(1, 9)] for r in range(1, 9)]]]


def ones(kh, kw):
    return [[[[1] * kw for _ in range(kh)]]]


w_c2 = [[[[1, 2], [3, 4]], [[4, 5], [6, 7]]]]


def conv(x, w, pv, ph, sv, sh, dv=1, dh=1):
    n, c, h, wd = len(x), len(x[0]), len(x[0][0]), len(x[0][0][0])
    kn, kh, kw = len(w), len(w[0][0]), len(w[0][0][0])
    ho = (h + 2 * pv - dv * (kh - 1) - 1) // sv + 1
    wo = (wd + 2 * ph - dh * (kw - 1) - 1) // sh + 1
    y = [[[[0] * wo for _ in range(ho)] for _ in range(kn)] for _ in range(n)]
    for nn in range(n):
        for co in range(kn):
            for oy in range(ho):
                for ox in range(wo):
                    acc = 0
                    for cc in range(c):
                        for i in range(kh):
                            for j in range(kw):
                                ih, iw = sv * oy + dv * i - pv, sh * ox + dh * j - ph
                                if 0 <= ih < h and 0 <= iw < wd:
                                    acc += w[co][cc][i][j] * x[nn][cc][ih][iw]
                    y[nn][co][oy][ox] = acc
    return y


cases = []
for name, x, w, geom in [
        ("x_2x4 * ones(2x2), no padding", x_2x4, ones(2, 2), (0, 0, 1, 1)),
        ("x_2x4 two channels * [[1,2],[3,4]],[[4,5],[6,7]], no padding", x_2x4_c2, w_c2, (0, 0, 1, 1)),
        ("x_2x4 * ones(1x1), padding 1", x_2x4, ones(1, 1), (1, 1, 1, 1)),
        ("x_2x4 * ones(1x2), padding 1", x_2x4, ones(1, 2), (1, 1, 1, 1)),
        ("x_4x4 * ones(2x2), padding 1, stride 2", x_4x4, ones(2, 2), (1, 1, 2, 2)),
        ("x_4x8 * ones(2x2), padding 1, stride (1,2)", x_4x8, ones(2, 2), (1, 1, 1, 2)),
        ("x_8x8 * ones(3x3), padding 1, stride 3", x_8x8, ones(3, 3), (1, 1, 3, 3)),
        ("x_8x8 * ones(2x2), padding 1", x_8x8, ones(2, 2), (1, 1, 1, 1)),
        ("x_8x8 * ones(3x3), padding 1, stride 2", x_8x8, ones(3, 3), (1, 1, 2, 2)),
        ("x_8x8 * ones(3x3), padding 2, dilation 2", x_8x8, ones(3, 3), (2, 2, 1, 1, 2, 2))]:
    cases.append({"name": name, "x": x, "w": w, "vpadding": geom[0], "hpadding": geom[1], "vstride": geom[2],
                  "hstride": geom[3], "vdilation": geom[4] if len(geom) > 4 else 1,
                  "hdilation": geom[5] if len(geom) > 5 else 1, "y": conv(x, w, *geom)})

assert cases[0]["y"] == [[[[51, 102, 204]]]]          # 1+2+16+32, 2+4+32+64, 4+8+64+128
# with the 1x3 bias matrix of pydtnn/tests/conv_gemm.py:151-155
cases[0]["bias_matrix"] = [[[[1024, 2048, 4196]]]]
cases[0]["y_plus_bias_matrix"] = [[[[1075, 2150, 4400]]]]

out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_hand_cases.json")
with open(out, "w") as f:
    json.dump({"layout": "NCHW; w is (kn, c, kh, kw)", "cases": cases}, f, indent=1)
print("wrote", out, len(cases), "cases")

"""Collect the reference's own golden vectors for the relax-star path into one JSON fixture.

Run in the build container (needs /root/reference, read-only):

    python tests/golden/extract_reference_vectors.py

Sources (data only; no reference code is imported or executed):
  * results/tests/baselines/set/test_star_affineMap_results.mat
      written by code/nnv/tests/set/star/test_star_affineMap.m:58-92
  * results/tests/baselines/set/star_test_results.mat
      written by code/nnv/tests/set/star/star_test.m
  * results/tests/baselines/nn/test_layers_relu_results.mat (IM_out) and the literals in
      code/nnv/tests/nn/layers/ReluLayer/test_layers_relu.m:19-33
  * results/tests/baselines/set/test_star_intersect_halfSpace_results.mat
      written by code/nnv/tests/set/star/test_star_intersect_halfSpace.m:66-79: a star with eleven
      general constraint rows and no predicate bounds, and its LP ranges (Star.getRanges)
  * results/tests/baselines/set/test_star_getBoxFast_results.mat
      written by code/nnv/tests/set/star/test_star_getBoxFast.m:10-63: a star over a random polytope,
      its LP box (Star.getBox, B1) and its interval box over the predicates' bounding box (getBoxFast, B2)
  * results/tests/baselines/set/test_star_isEmptySet_results.mat
      written by code/nnv/tests/set/star/test_star_isEmptySet.m:8-37: a feasible star over a random
      polytope (ten constraint rows) and the verdict Star.isEmptySet gave for it
  * the literal inputs/expected outputs typed in
      code/nnv/tests/nn/layers/Conv2DLayer/test_layers_Conv2D.m:14-28  (conv known answer)
      code/nnv/tests/set/image_star/test_ImageStar_getRange.m:45-62    (ranges known answer)
The .mat files are MATLAB v5 files read with scipy.io.loadmat (no code execution).
"""
import json
import os
import sys

import numpy as np
import scipy.io as sio

REF = "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "nnv_reference_vectors.json")


def arr(a):
    a = np.asarray(a, dtype=np.float64)
    return {"shape": list(a.shape), "data_colmajor": [float.hex(float(x)) for x in a.reshape(-1, order="F")]}


def main():
    if not os.path.isdir(REF):
        sys.exit("reference tree not mounted; the committed JSON is the fixture")
    out = {}
    base = os.path.join(REF, "results/tests/baselines")
    m = sio.loadmat(os.path.join(base, "set/test_star_affineMap_results.mat"))
    out["star_affineMap"] = {k: arr(m[k]) for k in
                             ("W", "b", "S_V", "S_C", "S_d", "S1_V", "S1_C", "S1_d", "W2", "S4_lb", "S4_ub")}
    out["star_affineMap"]["box_lb"] = arr([0, -1, 0])   # test_star_affineMap.m:59
    out["star_affineMap"]["box_ub"] = arr([1, 1, 1])    # test_star_affineMap.m:60
    m = sio.loadmat(os.path.join(base, "set/test_star_intersect_halfSpace_results.mat"))
    out["star_intersect_halfSpace"] = {k: arr(m[k]) for k in ("H", "g", "S_V", "S1_V", "S1_C", "S1_d", "S1_lb", "S1_ub")}
    m = sio.loadmat(os.path.join(base, "set/test_star_getBoxFast_results.mat"))
    out["star_getBoxFast"] = {k: arr(m[k]) for k in ("I1_V", "I1_C", "I1_d", "B1_lb", "B1_ub", "B2_lb", "B2_ub")}
    m = sio.loadmat(os.path.join(base, "set/test_star_isEmptySet_results.mat"))
    out["star_isEmptySet"] = {k: arr(m[k]) for k in ("S_V", "S_C", "S_d", "S1_V", "S1_C", "S1_d", "b_nonempty", "b_empty")}
    m = sio.loadmat(os.path.join(base, "set/star_test_results.mat"))
    out["star_test"] = {k: arr(m[k]) for k in ("S1_V", "S2_V", "S3_V", "B2_lb", "B2_ub")}
    # literal input / expected output of ReluLayer.evaluate typed in test_layers_relu.m:19-33
    # (the .mat baseline of that test keeps IM_out but a later, overwritten IM, so the source
    # literals are the input/output pair); IM_out is cross-checked against the .mat copy.
    IM = np.stack([np.array([[-1, 1, 0, -1], [0, 0, 1, -1], [1, 0, -1, 0], [1, -1, -1, 1]]),
                   np.array([[0, 1, 0, 0], [1, 0, 0, -1], [0, 1, -1, 0], [0, 1, 0, -1]]),
                   np.array([[1, -1, 1, 1], [1, -1, 0, 1], [0, 1, -1, 0], [1, 0, -1, 0]])], axis=2)
    IM_out = np.stack([np.array([[0, 1, 0, 0], [0, 0, 1, 0], [1, 0, 0, 0], [1, 0, 0, 1]]),
                       np.array([[0, 1, 0, 0], [1, 0, 0, 0], [0, 1, 0, 0], [0, 1, 0, 0]]),
                       np.array([[1, 0, 1, 1], [1, 0, 0, 1], [0, 1, 0, 0], [1, 0, 0, 0]])], axis=2)
    m = sio.loadmat(os.path.join(base, "nn/test_layers_relu_results.mat"))
    assert np.array_equal(m["IM_out"], IM_out)
    out["relu_evaluate"] = {"IM": arr(IM), "IM_out": arr(IM_out)}
    # literal known answers from the reference's test sources
    I = [[1, 1, 1, 0, 0], [0, 1, 1, 1, 0], [0, 0, 1, 1, 1], [0, 0, 1, 1, 0], [0, 1, 1, 0, 0]]
    W = [[1, 0, 1], [0, 1, 0], [1, 0, 1]]
    I_ = np.array(I, dtype=float)
    # the test's "checker" expression: sum of the five taps where W is 1
    chk = np.array([[I_[r, c] + I_[r, c + 2] + I_[r + 1, c + 1] + I_[r + 2, c] + I_[r + 2, c + 2]
                     for c in range(3)] for r in range(3)])
    out["conv2d_featureMap"] = {"I": arr(I), "W": arr(W), "padding": [0, 0, 0, 0], "stride": [1, 1],
                                "dilation": [1, 1], "expected": arr(chk)}
    out["imagestar_getRange_issue"] = {"V": arr(np.array([0.0, -1.0, 1.0]).reshape(1, 1, 1, 3)),
                                       "pred_lb": arr([-1, -1]), "pred_ub": arr([1, 1]),
                                       "expected_lb": arr([-2.0]), "expected_ub": arr([2.0])}
    with open(OUT, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", OUT)


if __name__ == "__main__":
    main()

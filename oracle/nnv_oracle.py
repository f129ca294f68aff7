"""CPU restatement of NNV's relax-star reachability path (TEST INFRASTRUCTURE ONLY).

This module is the *checker* for the HIP implementation.  It restates, statement by
statement and in fp64 numpy, what the MATLAB reference does on the path

    NN.reach -> {FullyConnectedLayer, Conv2DLayer, ReluLayer}.reach
             -> Star.affineMap / dlconv / PosLin.reach_relaxed_star_* (relaxFactor = 1)

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.  The
product (nnv_amd) never imports it and has no CPU fallback.

Conventions
-----------
* Matrices are numpy arrays; ``V`` is ``N x (n+1)`` with column 0 the centre, exactly as
  the reference's ``Star.V``.  Image tensors are ``H x W x C x (n+1)`` like ``ImageStar.V``
  and are flattened in MATLAB (column-major, ``order='F'``) order.
* Index vectors are 0-based here (the reference's are 1-based doubles).
* Every function cites the reference file:line (relative to code/nnv/engine/) it follows.

Parity pinning (what checks each function; see tests/test_oracle_*.py)
----------------------------------------------------------------------
* box_generators / star_from_box / affine_map / estimate_ranges: the reference's own
  golden file results/tests/baselines/set/test_star_affineMap_results.mat (S1_V, S4_lb,
  S4_ub), star_test_results.mat, the ImageStar getRange known answer ([-2, 2]) and the
  interval-arithmetic closed form.
* conv2d_feature_map / conv2d_reach: the reference's known-answer test
  tests/nn/layers/Conv2DLayer/test_layers_Conv2D.m:14-28, and torch's fp64 conv2d as an
  independent library routine.  Bit-level parity with MathWorks' closed ``dlconv``:
  PARITY UNPINNED (summation order unknowable here; values agree to rounding).
* box_partition: closed form (Cartesian grid, first listed index slowest).
* reach_relaxed_star / multiple_step_reach_star_approx_at_one: no reference test runs a
  relax-star method, so PARITY UNPINNED by golden vectors; pinned by the source text plus
  hand-computed scalar triangle, brute-force corner enumeration, the containment
  (soundness) invariant the reference's own soundness tests use, structural invariants
  and permutation-equivalence of the six variants.
* lpsolver / get_min(s) / get_max(s) / reach_relaxed_star_lp (relaxFactor < 1): the box-only branch of
  lpsolver is a closed form (checked against interval arithmetic); everything that reaches the LP
  solver is PARITY UNPINNED (linprog there, HiGHS here: values to solver tolerance, and a neuron whose
  optimised bound lies within that tolerance of 0 may be classified differently).  Pinned by: LP bounds never looser than estimateRanges, the rf = 1 limit (no LP), the box-star case where every
  variant reduces to the rf = 1 sets up to the documented order of the new predicates, and the
  containment invariant of the reference's soundness tests.  get_min / get_max through the solver
  branch are checked against the reference's stored LP ranges of a star with eleven general
  constraint rows (results/tests/baselines/set/test_star_intersect_halfSpace_results.mat, S1_lb /
  S1_ub, written by tests/set/star/test_star_intersect_halfSpace.m:66-79) and the stored Star.getBox of
  another (test_star_getBoxFast_results.mat, B1) to 1e-8; the same file's getBoxFast box (B2) is a second
  known answer for estimate_ranges' interval formula on a general V.
* halfspace_contains / is_empty_set / intersect_half_space: the reference's known answers
  (tests/set/halfspace/test_half_space_contain.m, tests/set/star/test_star_isEmptySet.m:17-23,
  tests/soundness/test_set_conversion.m:60-68) and closed forms on boxes.  The LP itself is
  MATLAB's linprog in the reference and scipy's HiGHS here: feasibility verdicts agree except
  within solver tolerance of the boundary.
* robustness_set / verify_specification: no reference test holds a value for them (the
  regression tests only check that the methods exist): PARITY UNPINNED by vectors; pinned by
  the source text, hand-built cases and the point-wise meaning of the verdict (a sampled
  output inside the unsafe region forces "unknown").
* avgpool2d_tensor: the reference's known answers without padding
  (tests/nn/layers/AveragePooling2DLayer/test_layers_averagePooling.m:14-23, 41-56) and, for the
  padded border, MatConvNet's published rule (mean over the cells inside the image) against torch's
  avg_pool2d(count_include_pad=False).  MatConvNet ships only as binaries in the reference:
  last-ulp summation order PARITY UNPINNED.
* batchnorm_*, image_input_*, image_star_affine_map, flatten_*: no reference test holds a value
  (PARITY UNPINNED by vectors); pinned by the textbook formulas, hand-computed permutations and by
  the affine-consistency identity reach(I).c = evaluate(c), reach(I).v_j = evaluate(c + v_j) -
  evaluate(c), which ties every reach restatement to its evaluate.
"""
from __future__ import annotations

import numpy as np

RELAX_METHODS = (
    "relax-star-range",
    "relax-star-area",
    "relax-star-bound",
    "relax-star-ub",
    "relax-star-random",
    "relax-star-static",
)


# --------------------------------------------------------------------------------------
# sets
# --------------------------------------------------------------------------------------
class OStar:
    """Field-for-field mirror of the reference's Star value class (set/Star.m:13-24)."""

    def __init__(self, V, C, d, predicate_lb=None, predicate_ub=None,
                 state_lb=None, state_ub=None, Z=None):
        # set/Star.m:153-189 (5-argument constructor and its size checks)
        V = np.asarray(V, dtype=np.float64)
        C = np.asarray(C, dtype=np.float64)
        d = np.asarray(d, dtype=np.float64).reshape(-1)
        if C.ndim != 2:
            C = C.reshape(-1, V.shape[1] - 1)
        if V.shape[1] != C.shape[1] + 1:
            raise ValueError("Inconsistency between basic matrix and constraint matrix")
        if C.shape[0] != d.shape[0]:
            raise ValueError("Inconsistency between constraint matrix and constraint vector")
        if predicate_lb is not None and predicate_ub is not None:
            predicate_lb = np.asarray(predicate_lb, dtype=np.float64).reshape(-1)
            predicate_ub = np.asarray(predicate_ub, dtype=np.float64).reshape(-1)
            if predicate_lb.size and predicate_ub.size and (
                    predicate_lb.size != predicate_ub.size or predicate_lb.size != C.shape[1]):
                raise ValueError("Inconsistency between number of predicate variables and "
                                 "predicate lower- or upper-bounds vector")
        self.V = V
        self.C = C
        self.d = d
        self.dim = V.shape[0]
        self.nVar = C.shape[1]
        self.predicate_lb = predicate_lb
        self.predicate_ub = predicate_ub
        self.state_lb = state_lb
        self.state_ub = state_ub
        self.Z = Z  # (c, V) of the outer zonotope or None


class OImageStar:
    """Mirror of the reference's ImageStar (set/ImageStar.m:47-94): V is H x W x C x (n+1)."""

    def __init__(self, V, C, d, pred_lb, pred_ub, im_lb=None, im_ub=None):
        # set/ImageStar.m:172-227 (5-argument constructor)
        V = np.asarray(V, dtype=np.float64)
        C = np.asarray(C, dtype=np.float64)
        d = np.asarray(d, dtype=np.float64).reshape(-1)
        if C.shape[0] != d.shape[0]:
            raise ValueError("Inconsistent dimension between constraint matrix and constraint vector")
        pred_lb = np.asarray(pred_lb, dtype=np.float64).reshape(-1)
        pred_ub = np.asarray(pred_ub, dtype=np.float64).reshape(-1)
        if C.shape[1] != pred_lb.size or C.shape[1] != pred_ub.size:
            raise ValueError("Number of predicates is different from the size of the lower "
                             "bound or upper bound predicate vector")
        if V.ndim != 4 or V.shape[3] != C.shape[1] + 1:
            raise ValueError("Inconsistency between the basis matrix and the number of predicate variables")
        self.V = V
        self.C = C
        self.d = d
        self.numPred = C.shape[1]
        self.pred_lb = pred_lb
        self.pred_ub = pred_ub
        self.height, self.width, self.numChannel = V.shape[:3]
        self.im_lb = im_lb
        self.im_ub = im_ub

    def to_star(self) -> OStar:
        # set/ImageStar.m:569-592: column j of the Star is reshape(V(:,:,:,j), N, 1)
        N = self.height * self.width * self.numChannel
        V1 = self.V.reshape(N, self.numPred + 1, order="F")
        if self.im_lb is not None and self.im_ub is not None:
            return OStar(V1, self.C, self.d, self.pred_lb, self.pred_ub,
                         np.asarray(self.im_lb).reshape(N, order="F"),
                         np.asarray(self.im_ub).reshape(N, order="F"))
        return OStar(V1, self.C, self.d, self.pred_lb, self.pred_ub)


def box_generators(lb, ub):
    """Box constructor arithmetic, set/Box.m:16-58.

    center = 0.5*(lb+ub); vec = 0.5*(ub-lb); generators = diag(vec) with all-zero columns
    removed (only when numel(gens) > 1, Box.m:41-43).
    """
    lb = np.asarray(lb, dtype=np.float64).reshape(-1)
    ub = np.asarray(ub, dtype=np.float64).reshape(-1)
    if lb.size != ub.size:
        raise ValueError("Inconsistent dimensions between lb and ub")
    center = 0.5 * (lb + ub)
    vec = 0.5 * (ub - lb)
    gens = np.diag(vec)
    if gens.size > 1:
        gens = gens[:, ~np.all(gens == 0, axis=0)]
    return center, gens


def box_single_partition(lb, ub, part_id, part_num):
    """set/Box.m:61-91 (part_id is 0-based here)."""
    if part_num == 1:
        return [(lb.copy(), ub.copy())]
    delta = (ub[part_id] - lb[part_id]) / part_num
    out = []
    for i in range(1, part_num + 1):
        new_lb = lb.copy()
        new_ub = ub.copy()
        new_lb[part_id] = lb[part_id] + (i - 1) * delta
        new_ub[part_id] = new_lb[part_id] + delta
        out.append((new_lb, new_ub))
    return out


def box_partition(lb, ub, part_indexes, part_numbers):
    """set/Box.m:96-139: successive single partitions; first listed index varies slowest."""
    lb = np.asarray(lb, dtype=np.float64).reshape(-1)
    ub = np.asarray(ub, dtype=np.float64).reshape(-1)
    boxes = [(lb, ub)]
    for idx, num in zip(part_indexes, part_numbers):
        nxt = []
        for (l, u) in boxes:
            nxt.extend(box_single_partition(l, u, idx, num))
        boxes = nxt
    return boxes


def star_from_box(lb, ub) -> OStar:
    """Star(lb, ub), set/Star.m:220-237 (+ Box.toStar -> Zono.toStar, set/Zono.m:301-309).

    V = [center gens]; C = zeros(1, n); d = 0; predicate bounds -1/+1; state bounds = lb/ub;
    Z = Zono(center, gens).
    """
    lb = np.asarray(lb, dtype=np.float64).reshape(-1)
    ub = np.asarray(ub, dtype=np.float64).reshape(-1)
    center, gens = box_generators(lb, ub)
    n = gens.shape[1]
    V = np.concatenate([center[:, None], gens], axis=1)
    return OStar(V, np.zeros((1, n)), np.zeros(1), -np.ones(n), np.ones(n),
                 lb.copy(), ub.copy(), Z=(center.copy(), gens.copy()))


def image_star_from_bounds(lb_im, ub_im) -> OImageStar:
    """ImageStar(lb_im, ub_im), set/ImageStar.m:302-343: Star(lb,ub).toImageStar(h,w,c)."""
    lb_im = np.asarray(lb_im, dtype=np.float64)
    ub_im = np.asarray(ub_im, dtype=np.float64)
    if lb_im.shape != ub_im.shape:
        raise ValueError("Inconsistency between lower bound image and upper bound image")
    if lb_im.ndim == 2:
        lb_im = lb_im[:, :, None]
        ub_im = ub_im[:, :, None]
    h, w, c = lb_im.shape
    S = star_from_box(lb_im.reshape(-1, order="F"), ub_im.reshape(-1, order="F"))
    IS = star_to_image_star(S, h, w, c)
    IS.im_lb = lb_im
    IS.im_ub = ub_im
    return IS


def star_to_image_star(S: OStar, height, width, num_channel) -> OImageStar:
    """Star.toImageStar, set/Star.m:1398-1418: plain column-major reshape of V."""
    if S.dim != height * width * num_channel:
        raise ValueError("Inconsistent dimension in the ImageStar and the original Star set")
    V = S.V.reshape(height, width, num_channel, S.nVar + 1, order="F")
    if S.state_lb is not None and S.state_ub is not None:
        return OImageStar(V, S.C, S.d, S.predicate_lb, S.predicate_ub,
                          np.asarray(S.state_lb).reshape(height, width, num_channel, order="F"),
                          np.asarray(S.state_ub).reshape(height, width, num_channel, order="F"))
    return OImageStar(V, S.C, S.d, S.predicate_lb, S.predicate_ub)


# --------------------------------------------------------------------------------------
# affine maps
# --------------------------------------------------------------------------------------
def affine_map(S: OStar, W, b=None) -> OStar:
    """Star.affineMap, set/Star.m:313-343.

    newV = W*V; newV(:,1) = newV(:,1) + b; C, d, predicate bounds pass through; the outer
    zonotope is mapped as well (set/Zono.m:47-74).  State bounds are dropped (6-arg ctor).
    """
    W = np.asarray(W, dtype=np.float64)
    if W.shape[1] != S.dim:
        raise ValueError("Inconsistency between the affine mapping matrix and dimension of the star set")
    newV = W @ S.V
    if b is not None and np.size(b):
        b = np.asarray(b, dtype=np.float64)
        if b.ndim == 2 and b.shape[1] != 1:
            raise ValueError("Mapping vector should have one column")
        b = b.reshape(-1)
        if b.shape[0] != W.shape[0]:
            raise ValueError("Inconsistency between the mapping vec and mapping matrix")
        newV[:, 0] = newV[:, 0] + b
    newZ = None
    if S.Z is not None:
        zc, zV = S.Z
        nc = W @ zc
        if b is not None and np.size(b):
            nc = nc + b
        newZ = (nc, W @ zV)
    return OStar(newV, S.C, S.d, S.predicate_lb, S.predicate_ub, Z=newZ)


def fc_reach(I, W, b):
    """FullyConnectedLayer.reach_star_single_input, nn/layers/FullyConnectedLayer.m:295-316, 467-481.

    ImageStar: V(1,1,:,:) = W*reshape(V, N, n+1); V(1,1,:,1) += Bias -> ImageStar 1x1xOutx(n+1).
    Star: affineMap(W, b).
    """
    W = np.asarray(W, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64).reshape(-1)
    if isinstance(I, OImageStar):
        N = I.height * I.width * I.numChannel
        if N != W.shape[1]:
            raise ValueError("Inconsistency between the size of the input image and the InputSize of the network")
        n = I.numPred
        newV = W @ I.V.reshape(N, n + 1, order="F")
        newV[:, 0] = newV[:, 0] + b
        return OImageStar(newV.reshape(1, 1, W.shape[0], n + 1, order="F"),
                          I.C, I.d, I.pred_lb, I.pred_ub)
    if isinstance(I, OStar):
        return affine_map(I, W, b)
    raise TypeError("Input set is not an ImageStar or Star")


def conv2d_output_size(H, W, FH, FW, padding, stride, dilation):
    """Feature-map size, nn/layers/Conv2DLayer.m:1134-1135 (padding = [t b l r])."""
    t, b, l, r = padding
    ho = int(np.floor((H + t + b - (FH - 1) * dilation[0] - 1) / stride[0] + 1))
    wo = int(np.floor((W + l + r - (FW - 1) * dilation[1] - 1) / stride[1] + 1))
    return ho, wo


def conv2d_feature_map(inp, Wf, padding, stride, dilation):
    """Conv2DLayer.compute_featureMap, nn/layers/Conv2DLayer.m:1111-1204 (single channel, 2-D).

    Zero padding [t b l r] (get_zero_padding_input, :1064-1108), then for every output cell
    val = sum_{i,j} I(i0 + (i-1)*dil, j0 + (j-1)*dil) * W(i,j): cross-correlation, no flip.
    Pure-python loops: used for small known-answer checks only.
    """
    inp = np.asarray(inp, dtype=np.float64)
    Wf = np.asarray(Wf, dtype=np.float64)
    t, b, l, r = padding
    h, w = inp.shape
    I = np.zeros((t + h + b, l + w + r))
    I[t:t + h, l:l + w] = inp
    ho, wo = conv2d_output_size(h, w, Wf.shape[0], Wf.shape[1], padding, stride, dilation)
    out = np.zeros((ho, wo))
    for i in range(ho):
        for j in range(wo):
            val = 0.0
            for fi in range(Wf.shape[0]):
                for fj in range(Wf.shape[1]):
                    ie = i * stride[0] + fi * dilation[0]
                    je = j * stride[1] + fj * dilation[1]
                    if ie < I.shape[0] and je < I.shape[1]:
                        val = val + I[ie, je] * Wf[fi, fj]
            out[i, j] = val
    return out


def conv2d_tensor(X, Wt, bias, padding, stride, dilation):
    """dlconv semantics used at nn/layers/Conv2DLayer.m:591-592 on an H x W x Cin x B tensor.

    Wt is FH x FW x Cin x Cout, cross-correlation (same definition as compute_featureMap
    summed over input channels), zero padding [t b l r].  bias (Cout,) or None is added after
    the sum.  Taps are accumulated in (fh fastest, fw, then the channel contraction) order.
    """
    X = np.asarray(X, dtype=np.float64)
    Wt = np.asarray(Wt, dtype=np.float64)
    H, W_, Cin, B = X.shape
    FH, FW, Cin2, Cout = Wt.shape
    if Cin != Cin2:
        raise ValueError("Input set contains %d channels while the convolutional layers has %d channels"
                         % (Cin, Cin2))
    t, b, l, r = padding
    ho, wo = conv2d_output_size(H, W_, FH, FW, padding, stride, dilation)
    Xp = np.zeros((t + H + b, l + W_ + r, Cin, B))
    Xp[t:t + H, l:l + W_] = X
    out = np.zeros((ho, wo, Cout, B))
    for fw in range(FW):
        for fh in range(FH):
            h0 = fh * dilation[0]
            w0 = fw * dilation[1]
            patch = Xp[h0:h0 + (ho - 1) * stride[0] + 1:stride[0],
                       w0:w0 + (wo - 1) * stride[1] + 1:stride[1]]  # ho x wo x Cin x B
            # contract the channel axis: (ho,wo,Cin,B) x (Cin,Cout) -> (ho,wo,Cout,B)
            out += np.einsum("hwcb,co->hwob", patch, Wt[fh, fw], optimize=True)
    if bias is not None:
        out += np.asarray(bias, dtype=np.float64).reshape(1, 1, Cout, 1)
    return out


def conv2d_reach(I: OImageStar, Wt, bias, padding=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1)) -> OImageStar:
    """Conv2DLayer.reach_star_single_input, nn/layers/Conv2DLayer.m:559-601, 780.

    c = dlconv(V(:,:,:,1), W, Bias); G = dlconv(V(:,:,:,2:end), W, 0); V' = cat(4, c, G);
    C, d, predicate bounds pass through; the result is a 5-argument ImageStar (no im_lb/ub).
    """
    if not isinstance(I, OImageStar):
        raise TypeError("The input is not an ImageStar object")
    Wt = np.asarray(Wt, dtype=np.float64)
    if I.numChannel != Wt.shape[2]:
        raise ValueError("Input set contains %d channels while the convolutional layers has %d channels"
                         % (I.numChannel, Wt.shape[2]))
    bias = np.zeros(Wt.shape[3]) if bias is None else np.asarray(bias, dtype=np.float64).reshape(-1)
    c = conv2d_tensor(I.V[:, :, :, :1], Wt, bias, padding, stride, dilation)
    G = conv2d_tensor(I.V[:, :, :, 1:], Wt, None, padding, stride, dilation)
    return OImageStar(np.concatenate([c, G], axis=3), I.C, I.d, I.pred_lb, I.pred_ub)


# --------------------------------------------------------------------------------------
# ranges and the relaxed ReLU
# --------------------------------------------------------------------------------------
def estimate_ranges(S: OStar):
    """Star.estimateRanges, set/Star.m:1078-1106.

    pos = max(V,0); neg = min(V,0) (whole matrix, centre column included); the four products
    use [0; predicate bounds] so the centre column cancels;
    lb = V(:,1) + xmin1 + xmin2, ub = V(:,1) + xmax1 + xmax2 (left to right).
    Empty predicate bounds default to -1/+1 (:1091-1096).
    """
    pos_mat = S.V.copy()
    neg_mat = S.V.copy()
    pos_mat[pos_mat < 0] = 0
    neg_mat[neg_mat > 0] = 0
    plb = S.predicate_lb
    pub = S.predicate_ub
    if plb is None or np.size(plb) == 0:
        plb = -np.ones(S.nVar)
    if pub is None or np.size(pub) == 0:
        pub = np.ones(S.nVar)
    lbv = np.concatenate([[0.0], plb])
    ubv = np.concatenate([[0.0], pub])
    xmin1 = pos_mat @ lbv
    xmax1 = pos_mat @ ubv
    xmin2 = neg_mat @ ubv
    xmax2 = neg_mat @ lbv
    lb = S.V[:, 0] + xmin1 + xmin2
    ub = S.V[:, 0] + xmax1 + xmax2
    return lb, ub


def image_star_estimate_ranges(I: OImageStar):
    """ImageStar.estimateRanges, set/ImageStar.m:836-885 (same formula on the tensor form)."""
    if I.im_lb is not None and I.im_ub is not None:
        return I.im_lb, I.im_ub
    gens = I.V[:, :, :, 1:]
    pos = np.where(gens < 0, 0.0, gens)
    neg = np.where(gens > 0, 0.0, gens)
    lb = I.V[:, :, :, 0] + np.tensordot(pos, I.pred_lb, axes=(3, 0)) + np.tensordot(neg, I.pred_ub, axes=(3, 0))
    ub = I.V[:, :, :, 0] + np.tensordot(pos, I.pred_ub, axes=(3, 0)) + np.tensordot(neg, I.pred_lb, axes=(3, 0))
    return lb, ub


def reset_row(S: OStar, rows) -> OStar:
    """Star.resetRow, set/Star.m:1442-1461: V(map,:) = 0 (and the same on Z)."""
    V1 = S.V.copy()
    V1[rows, :] = 0
    newZ = None
    if S.Z is not None:
        c2 = S.Z[0].copy()
        c2[rows] = 0
        V2 = S.Z[1].copy()
        V2[rows, :] = 0
        newZ = (c2, V2)
    return OStar(V1, S.C, S.d, S.predicate_lb, S.predicate_ub, Z=newZ)


def multiple_step_reach_star_approx_at_one(I: OStar, index, lb, ub) -> OStar:
    """PosLin.multipleStepReachStarApprox_at_one, nn/funcs/PosLin.m:685-742.

    index: crossing neurons (0-based) in the order the new predicate columns get; lb/ub their
    bounds.  Returns Star(new_V, new_C, new_d, new_pred_lb, new_pred_ub): no Z, no state bounds.
    """
    index = np.asarray(index, dtype=np.int64).reshape(-1)
    lb = np.asarray(lb, dtype=np.float64).reshape(-1)
    ub = np.asarray(ub, dtype=np.float64).reshape(-1)
    N = I.dim
    m = index.size
    V1 = I.V.copy()
    V1[index, :] = 0
    V2 = np.zeros((N, m))
    for i in range(m):
        V2[index[i], i] = 1
    new_V = np.concatenate([V1, V2], axis=1)

    n = I.nVar
    C0 = np.concatenate([I.C, np.zeros((I.C.shape[0], m))], axis=1)
    d0 = I.d
    C1 = np.concatenate([np.zeros((m, n)), -np.eye(m)], axis=1)
    d1 = np.zeros(m)
    C2 = np.concatenate([I.V[index, 1:n + 1], -V2[index, :m]], axis=1)
    d2 = -I.V[index, 0]
    a = ub / (ub - lb)
    b = a * lb
    C3 = np.concatenate([(-a)[:, None] * I.V[index, 1:n + 1], V2[index, :m]], axis=1)
    d3 = a * I.V[index, 0] - b
    new_C = np.concatenate([C0, C1, C2, C3], axis=0)
    new_d = np.concatenate([d0, d1, d2, d3])
    new_pred_lb = np.concatenate([I.predicate_lb, np.zeros(m)])
    new_pred_ub = np.concatenate([I.predicate_ub, ub])
    return OStar(new_V, new_C, new_d, new_pred_lb, new_pred_ub)


def relax_classify(lb, ub, method):
    """Classification and crossing order shared by the six variants at relaxFactor = 1.

    map1 = find(ub <= 0); map2 = find(lb < 0 & ub > 0) (ascending);
    range: sort(ub-lb,'descend') (nn/funcs/PosLin.m:934-936);
    area:  sort(0.5*(abs(ub).*abs(lb)),'descend') (:1049-1052);
    bound/ub/random/static keep ascending order (:1167-1174,1232; :1326-1329,1397;
    :1488-1492; :1604-1605).  MATLAB's sort is stable.
    """
    map1 = np.flatnonzero(ub <= 0)
    map2 = np.flatnonzero((lb < 0) & (ub > 0))
    if method == "relax-star-range":
        key = ub[map2] - lb[map2]
        order = np.argsort(-key, kind="stable")
        map2 = map2[order]
    elif method == "relax-star-area":
        key = 0.5 * (np.abs(ub[map2]) * np.abs(lb[map2]))
        order = np.argsort(-key, kind="stable")
        map2 = map2[order]
    elif method not in RELAX_METHODS:
        raise ValueError("This reachability method does not exist")
    return map1, map2


def lpsolver(f, A, b, lb, ub):
    """utils/lpsolver.m: min f'x s.t. A x <= b, lb <= x <= ub -> fval.

    The box-only shortcut (:36-50: A empty or all-zero, finite bounds, b >= 0) is restated exactly:
    fval = sum(min(f.*lb, f.*ub)).  Otherwise MATLAB's linprog (glpk as backup) is replaced by
    scipy's HiGHS, so values agree to solver tolerance only: PARITY UNPINNED beyond that."""
    f = np.asarray(f, dtype=np.float64).reshape(-1)
    A = np.asarray(A, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64).reshape(-1)
    if (A.size == 0 or not np.any(A)) and lb is not None and ub is not None and np.size(lb) and np.size(ub) \
            and np.all(np.isfinite(lb)) and np.all(np.isfinite(ub)) and (b.size == 0 or np.all(b >= 0)):
        return float(np.sum(np.minimum(f * lb, f * ub)))
    from scipy.optimize import linprog
    n = f.size
    lo = np.full(n, -np.inf) if lb is None or not np.size(lb) else np.asarray(lb, dtype=np.float64).reshape(-1)
    hi = np.full(n, np.inf) if ub is None or not np.size(ub) else np.asarray(ub, dtype=np.float64).reshape(-1)
    res = linprog(f, A_ub=A if A.size else None, b_ub=b if A.size else None,
                  bounds=np.column_stack([lo, hi]), method="highs")
    if res.status != 0:
        raise RuntimeError("Cannot find an optimal solution, exitflag = %d" % res.status)
    return float(res.fun)


def get_min(S: OStar, index) -> float:
    """Star.getMin, set/Star.m:744-781 (index 0-based): the centre entry if the generator row is all
    zero, else one LP over (C, d, predicate bounds)."""
    if index < 0 or index >= S.dim:
        raise ValueError("Invalid index")
    f = S.V[index, 1:S.nVar + 1]
    if not np.any(f):
        return float(S.V[index, 0])
    return lpsolver(f, S.C, S.d, S.predicate_lb, S.predicate_ub) + float(S.V[index, 0])


def get_max(S: OStar, index) -> float:
    """Star.getMax, set/Star.m:859-895: -min(-f) + c."""
    if index < 0 or index >= S.dim:
        raise ValueError("Invalid index")
    f = S.V[index, 1:S.nVar + 1]
    if not np.any(f):
        return float(S.V[index, 0])
    return -lpsolver(-f, S.C, S.d, S.predicate_lb, S.predicate_ub) + float(S.V[index, 0])


def get_mins(S: OStar, idx):
    """Star.getMins, set/Star.m:784-856 (single-core branch)."""
    return np.array([get_min(S, int(i)) for i in np.asarray(idx).reshape(-1)], dtype=np.float64)


def get_maxs(S: OStar, idx):
    """Star.getMaxs, set/Star.m:898-970."""
    return np.array([get_max(S, int(i)) for i in np.asarray(idx).reshape(-1)], dtype=np.float64)


def _round_half_away(x):
    return int(np.floor(x + 0.5))  # MATLAB round() for x >= 0


def _setdiff_stable(a, b):
    """setdiff(a, b, 'stable') for index vectors."""
    b = set(int(v) for v in np.asarray(b).reshape(-1))
    return np.array([v for v in np.asarray(a).reshape(-1) if int(v) not in b], dtype=np.int64)


def reach_relaxed_star_lp(I: OStar, method: str, relax_factor: float, rng=None) -> OStar:
    """PosLin.reach_relaxed_star_{range,area,random,static} (nn/funcs/PosLin.m:863-983, 986-1104,
    1425-1538, 1541-1650) and _{bound,ub} (:1107-1260, :1263-1422) for any relaxFactor:
    n1 = round((1-rf)*numel(map2)) neurons get LP bounds.  Statement order follows the source."""
    lb, ub = estimate_ranges(I)
    map1 = np.flatnonzero(ub <= 0)
    map2 = np.flatnonzero((lb < 0) & (ub > 0))
    n1 = _round_half_away((1 - relax_factor) * map2.size)
    if method in ("relax-star-range", "relax-star-area", "relax-star-random", "relax-star-static"):
        if method == "relax-star-range":
            midx = np.argsort(-(ub[map2] - lb[map2]), kind="stable")
            map21, map22 = map2[midx[:n1]], map2[midx[n1:]]
        elif method == "relax-star-area":
            areas = 0.5 * (np.abs(ub[map2]) * np.abs(lb[map2]))
            midx = np.argsort(-areas, kind="stable")
            map21, map22 = map2[midx[:n1]], map2[midx[n1:]]
        elif method == "relax-star-random":
            midx = (rng or np.random).permutation(map2.size)[:n1]   # randperm(length(map2), n1)
            map21 = map2[midx]
            map22 = _setdiff_stable(map2, map21)
        else:
            map21, map22 = map2[:n1], map2[n1:]
        lb1, ub1 = lb[map22], ub[map22]
        xmax = get_maxs(I, map21)
        map3 = np.flatnonzero(xmax <= 0)
        map4 = map21[map3]
        map11 = np.concatenate([map1, map4]).astype(np.int64)
        In = reset_row(I, map11)
        map5 = np.flatnonzero(xmax > 0)
        map6 = map21[map5]
        xmax1 = xmax[map5]
        xmin = get_mins(I, map6)
        map7 = np.flatnonzero(xmin < 0)
        map8 = map6[map7]
        lb2, ub2 = xmin[map7], xmax1[map7]
        map9 = np.concatenate([map22, map8]).astype(np.int64)
        lb3 = np.concatenate([lb1, lb2])
        ub3 = np.concatenate([ub1, ub2])
        return multiple_step_reach_star_approx_at_one(In, map9, lb3, ub3)
    if method not in ("relax-star-bound", "relax-star-ub"):
        raise ValueError("This reachability method does not exist")
    N = map2.size
    if method == "relax-star-bound":
        lu = np.concatenate([ub[map2], np.abs(lb[map2])])
        midx = np.argsort(-lu, kind="stable")
        midx1 = midx[:2 * n1]
        ub_idx = midx1[midx1 < N]
        lb_idx = midx1[midx1 >= N] - N
        map21, map22 = map2[ub_idx], map2[lb_idx]
    else:
        midx_u = np.argsort(-ub[map2], kind="stable")
        midx_l = np.argsort(-np.abs(lb[map2]), kind="stable")
        if 2 * n1 <= N:
            map21, map22 = map2[midx_u[:2 * n1]], np.zeros(0, dtype=np.int64)
        else:
            map21, map22 = map2[midx_u[:N]], map2[midx_l[:2 * n1 - N]]
    lb, ub = lb.copy(), ub.copy()
    if map21.size:
        xmax = get_maxs(I, map21)
        map4 = map21[np.flatnonzero(xmax <= 0)]
        map5 = np.flatnonzero(xmax > 0)
        map6 = map21[map5]
        map11 = np.concatenate([map1, map4]).astype(np.int64)
    else:
        map11, map5, map6, map4 = map1, np.zeros(0, dtype=np.int64), np.zeros(0, dtype=np.int64), np.zeros(0, dtype=np.int64)
    In = reset_row(I, map11)
    map23 = _setdiff_stable(map22, map4) if map4.size else map22
    if map23.size:
        xmin = get_mins(I, map23)
        map7 = np.flatnonzero(xmin < 0)
        map8 = map23[map7]
        map10 = map23[np.flatnonzero(xmin >= 0)]
    else:
        map7, map8, map10 = np.zeros(0, dtype=np.int64), np.zeros(0, dtype=np.int64), np.zeros(0, dtype=np.int64)
    map24 = _setdiff_stable(map2, map4) if map4.size else map2
    if map10.size:
        map24 = _setdiff_stable(map24, map10)
    if map6.size:
        ub[map6] = xmax[map5]
    if map8.size:
        lb[map8] = xmin[map7]
    return multiple_step_reach_star_approx_at_one(In, map24, lb[map24], ub[map24])


def reach_relaxed_star(I: OStar, method: str, relax_factor: float = 1.0, rng=None) -> OStar:
    """PosLin.reach_relaxed_star_{range,area,bound,ub,random,static} (nn/funcs/PosLin.m:863-1650).
    At relaxFactor = 1, n1 = round((1-rf)*numel(map2)) = 0 and no LP is solved:
    In = I.resetRow(map1); S = multipleStepReachStarApprox_at_one(In, map, lb(map), ub(map));
    below 1 see reach_relaxed_star_lp."""
    if not isinstance(I, OStar):
        raise TypeError("Input is not a star")
    if relax_factor < 0 or relax_factor > 1:
        raise ValueError("Invalid relax factor")
    if method not in RELAX_METHODS:
        raise ValueError("This reachability method does not exist")
    if relax_factor != 1:
        return reach_relaxed_star_lp(I, method, relax_factor, rng)
    lb, ub = estimate_ranges(I)
    map1, mp = relax_classify(lb, ub, method)
    In = reset_row(I, map1)
    return multiple_step_reach_star_approx_at_one(In, mp, lb[mp], ub[mp])


def poslin_reach(I, method, option=None, relax_factor=0.0, dis_opt=None, lp_solver="linprog"):
    """PosLin.reach dispatcher, nn/funcs/PosLin.m:2073-2169 (relax-star branches only)."""
    if method in RELAX_METHODS:
        return reach_relaxed_star(I, method, relax_factor)
    raise ValueError("This reachability method does not exist")


def relu_reach(I, method, relax_factor=1.0):
    """ReluLayer.reach_star_single_input, nn/layers/ReluLayer.m:72-150.

    ImageStar: toStar -> PosLin.reach -> toImageStar(h, w, c); Star: PosLin.reach.
    """
    if isinstance(I, OImageStar):
        Y = poslin_reach(I.to_star(), method, None, relax_factor)
        return star_to_image_star(Y, I.height, I.width, I.numChannel)
    if isinstance(I, OStar):
        return poslin_reach(I, method, None, relax_factor)
    raise TypeError("input is not an ImageStar, Star or VolumeStar")


# --------------------------------------------------------------------------------------
# network loop
# --------------------------------------------------------------------------------------
def relu_reduce_mem(I: OImageStar) -> OImageStar:
    """The reduceMem suffix of ReluLayer.reach_star_single_input, nn/layers/ReluLayer.m:119-146, statement
    for statement: the ReLU's output ImageStar is replaced by a box-like ImageStar built from its estimated
    ranges.  n counts every element with l ~= u; a generator is made per PIXEL (i1 outer, i2 inner) whose
    first-channel half-width v(i1,i2) is non-zero, and that value is written to every channel of the pixel
    (V(i1,i2,:,bCount) = v(i1,i2)); generators that are never filled stay zero."""
    l, u = image_star_estimate_ranges(I)
    l = np.asarray(l, dtype=np.float64)
    u = np.asarray(u, dtype=np.float64)
    h, w, c = I.height, I.width, I.numChannel
    center = 0.5 * (u + l)
    v = 0.5 * (u - l)
    n = int(np.count_nonzero(l - u))            # idxRegion = find((l-u)); n = length(idxRegion)
    V = np.zeros((h, w, c, n))
    b_count = 0
    for i1 in range(h):
        for i2 in range(w):
            basis = v[i1, i2, 0]                # v(i1,i2) of a 3-D array is v(i1,i2,1)
            if basis:
                V[i1, i2, :, b_count] = basis
                b_count += 1
    Cm = np.zeros((1, n))
    d = np.zeros(1)
    return OImageStar(np.concatenate([center[:, :, :, None], V], axis=3), Cm, d, -np.ones(n), np.ones(n), l, u)


def relu_layer_reach(I, method, relax_factor=1.0):
    """ReluLayer.reach_star_single_input, nn/layers/ReluLayer.m:72-150, for a Star or an ImageStar: the
    'reduceMem' suffix is split off the method for ImageStars only (:107-112); a Star hands the whole string
    to PosLin.reach, which does not know it (nn/funcs/PosLin.m:2165-2166)."""
    if isinstance(I, OImageStar):
        reduce_mem = "reduceMem" in method
        if reduce_mem:
            method = "-".join(method.split("-")[:-1])
        R = relu_reach(I, method, relax_factor)
        return relu_reduce_mem(R) if reduce_mem else R
    if "reduceMem" in method:
        raise ValueError("This reachability method does not exist")
    return relu_reach(I, method, relax_factor)


def nn_reach(layers, input_set, reach_method="relax-star-area", relax_factor=1.0, keep=False):
    """NN.reach -> reach_noConns, nn/NN.m:189-278, 1529-1551, for a list of layer dicts:

    {"type": "fc", "W": (Out x In), "b": (Out,)}
    {"type": "conv", "W": (FH x FW x Cin x Cout), "b": (Cout,), "padding": [t b l r],
     "stride": [sh sw], "dilation": [dh dw]}
    {"type": "relu"}

    input_set may be a set or a list of sets (the reference loops serially over arrays,
    nn/layers/FullyConnectedLayer.m:504-507).  Returns the output set(s); with keep=True also
    the per-layer sets (NN.reachSet).
    """
    if "relax-star" in reach_method and not (0 <= relax_factor <= 1):
        raise ValueError("Invalid relaxFactor. The value of relax factor must be between 0 and 1")
    single = not isinstance(input_set, (list, tuple))
    sets = [input_set] if single else list(input_set)
    reach_set = []
    for L in layers:
        out = []
        for S in sets:
            if L["type"] == "fc":
                out.append(fc_reach(S, L["W"], L["b"]))
            elif L["type"] == "conv":
                out.append(conv2d_reach(S, L["W"], L.get("b"), L.get("padding", (0, 0, 0, 0)),
                                        L.get("stride", (1, 1)), L.get("dilation", (1, 1))))
            elif L["type"] == "relu":
                out.append(relu_layer_reach(S, reach_method, relax_factor))
            elif L["type"] == "batchnorm":
                out.append(batchnorm_reach(S, L["mean"], L["var"], L["eps"], L["scale"], L["offset"]))
            elif L["type"] == "avgpool":
                out.append(avgpool2d_reach(S, L["pool"], L["stride"], L["padding"]))
            elif L["type"] == "flatten":
                out.append(flatten_reach(S, L["flatten_type"]))
            elif L["type"] == "imageinput":
                out.append(image_input_reach(S, L["normalization"], L.get("mean"), L.get("std"), L.get("min"), L.get("max")))
            elif L["type"] == "layers":
                out.append(layers_reach(S, L["W"], L["b"], L["f"], reach_method, relax_factor))
            else:
                raise ValueError("unknown layer type " + str(L["type"]))
        sets = out
        if keep:
            reach_set.append(out[0] if single else out)
    res = sets[0] if single else sets
    return (res, reach_set) if keep else res


def output_ranges(S):
    """Reported output bounds: estimateRanges of the last layer's set (set/Star.m:1078-1106)."""
    if isinstance(S, OImageStar):
        S = S.to_star() if S.im_lb is None else OStar(
            S.V.reshape(-1, S.numPred + 1, order="F"), S.C, S.d, S.pred_lb, S.pred_ub)
    return estimate_ranges(S)


def evaluate(layers, x):
    """Concrete forward pass (layer.evaluate) used by the containment checks:
    FC y = W*x + b (nn/layers/FullyConnectedLayer.m:159), conv = cross-correlation + bias,
    ReLU = max(x, 0)."""
    x = np.asarray(x, dtype=np.float64)
    for L in layers:
        if L["type"] == "fc":
            x = np.asarray(L["W"]) @ x.reshape(-1, order="F") + np.asarray(L["b"]).reshape(-1)
        elif L["type"] == "conv":
            x = conv2d_tensor(x.reshape(x.shape + (1,) * (4 - x.ndim)) if x.ndim == 3 else x[:, :, None, None],
                              L["W"], L.get("b"), L.get("padding", (0, 0, 0, 0)),
                              L.get("stride", (1, 1)), L.get("dilation", (1, 1)))[:, :, :, 0]
        elif L["type"] == "relu":
            x = np.maximum(x, 0)
        elif L["type"] == "batchnorm":
            x = batchnorm_evaluate(x, L["mean"], L["var"], L["eps"], L["scale"], L["offset"])
        elif L["type"] == "avgpool":
            x = avgpool2d_tensor(x[:, :, :, None], L["pool"], L["stride"], L["padding"])[:, :, :, 0]
        elif L["type"] == "flatten":
            x = flatten_evaluate(x, L["flatten_type"]) if x.ndim == 3 else x
        elif L["type"] == "imageinput":
            x = image_input_evaluate(x, L["normalization"], L.get("mean"), L.get("std"), L.get("min"), L.get("max"))
        elif L["type"] == "layers":
            x = np.asarray(L["W"]) @ x.reshape(-1, order="F") + np.asarray(L["b"]).reshape(-1)
            if L["f"] == "poslin":
                x = np.maximum(x, 0)
    return x


# --------------------------------------------------------------------------------------
# further affine layers: batch normalisation, average pooling, flatten, input normalisation
# --------------------------------------------------------------------------------------
def _chan(a, C):
    """A per-channel parameter (1x1xC array, vector or scalar) as a length-C vector."""
    a = np.asarray(a, dtype=np.float64).reshape(-1)
    if a.size == 1:
        a = np.repeat(a, C)
    if a.size != C:
        raise ValueError("Inconsistent number of channels between scale array and the ImageStar")
    return a


def batchnorm_evaluate(x, mean, var, eps, scale, offset):
    """BatchNormalizationLayer.evaluate, nn/layers/BatchNormalizationLayer.m:118-229: per channel
    (third axis of an image, entries of a vector) ((x - mean)/sqrt(var + eps))*scale + offset."""
    x = np.asarray(x, dtype=np.float64)
    if x.ndim == 3:
        C = x.shape[2]
        m, v, s, o = (_chan(a, C)[None, None, :] for a in (mean, var, scale, offset))
    else:
        C = x.size
        m, v, s, o = (_chan(a, C).reshape(x.shape) for a in (mean, var, scale, offset))
    return s * ((x - m) / np.sqrt(v + eps)) + o


def batchnorm_reach(I, mean, var, eps, scale, offset):
    """BatchNormalizationLayer.reach_star_single_input, nn/layers/BatchNormalizationLayer.m:247-351.

    ImageStar (:286-330), per channel i:  V(:,:,i,1) -= mean_i;  V(:,:,i,:) = V(:,:,i,:) .* 1 / sqrt(var_i + eps)
    (MATLAB evaluates `x .* 1 / s` left to right: a division by s);  V(:,:,i,:) .*= scale_i;
    V(:,:,i,1) += offset_i.   Star (:332-349):  l = scale ./ sqrt(var + eps);  b = offset - mean .* l;
    V = V .* l;  V(:,1) += b."""
    if isinstance(I, OImageStar):
        C = I.numChannel
        m, v, s, o = (_chan(a, C) for a in (mean, var, scale, offset))
        V = I.V.copy()
        for i in range(C):
            V[:, :, i, 0] = V[:, :, i, 0] - m[i]
            V[:, :, i, :] = (V[:, :, i, :] * 1.0) / np.sqrt(v[i] + eps)
            V[:, :, i, :] = V[:, :, i, :] * s[i]
            V[:, :, i, 0] = V[:, :, i, 0] + o[i]
        return OImageStar(V, I.C, I.d, I.pred_lb, I.pred_ub)
    if isinstance(I, OStar):
        N = I.dim
        m, v, s, o = (_chan(a, N) for a in (mean, var, scale, offset))
        l = s / np.sqrt(v + eps)
        b = o - m * l
        V = I.V * l[:, None]
        V[:, 0] = V[:, 0] + b
        return OStar(V, I.C, I.d, I.predicate_lb, I.predicate_ub)
    raise TypeError("Input is not a Star, ImageStar or VolumeStar")


def avgpool2d_output_size(H, W, pool, padding, stride):
    """AveragePooling2DLayer.get_size_averageMap, nn/layers/AveragePooling2DLayer.m:396-418."""
    t, b, l, r = padding
    return ((H + t + b - pool[0]) // stride[0] + 1, (W + l + r - pool[1]) // stride[1] + 1)


def avgpool2d_tensor(X, pool, stride, padding):
    """AveragePooling2DLayer.evaluate, nn/layers/AveragePooling2DLayer.m:229-247 = MatConvNet's
    vl_nnpool(..., 'Method', 'avg') (third-party, vendored only as binaries; restated from its
    published CPU source): for every output cell the window is clipped to the image and the mean is
    taken over the cells that remain (padding does not count), as sum * (1 / count); the sum runs
    over window columns (outer) and rows (inner).  X: H x W x C x B."""
    X = np.asarray(X, dtype=np.float64)
    H, W, C, B = X.shape
    ph, pw = pool
    sh, sw = stride
    t, b, l, r = padding
    Ho, Wo = avgpool2d_output_size(H, W, pool, padding, stride)
    Y = np.zeros((Ho, Wo, C, B))
    for wo in range(Wo):
        x1 = wo * sw - l
        x2 = min(x1 + pw, W)
        x1 = max(x1, 0)
        for ho in range(Ho):
            y1 = ho * sh - t
            y2 = min(y1 + ph, H)
            y1 = max(y1, 0)
            acc = np.zeros((C, B))
            for x in range(x1, x2):
                for y in range(y1, y2):
                    acc = acc + X[y, x, :, :]
            Y[ho, wo, :, :] = acc * (1.0 / ((y2 - y1) * (x2 - x1)))
    return Y


def avgpool2d_reach(I: OImageStar, pool, stride, padding) -> OImageStar:
    """AveragePooling2DLayer.reach_star_single_input, nn/layers/AveragePooling2DLayer.m:424-436:
    Y = evaluate(V) on all n+1 images; constraints and predicate bounds unchanged."""
    if not isinstance(I, OImageStar):
        raise TypeError("The input is not an ImageStar object")
    return OImageStar(avgpool2d_tensor(I.V, pool, stride, padding), I.C, I.d, I.pred_lb, I.pred_ub)


def flatten_evaluate(image, layer_type):
    """FlattenLayer.evaluate for an H x W x C image, nn/layers/FlattenLayer.m:118-170: MATLAB style is
    a column-major reshape; Keras C-style permutes [3 2 1] first; the ONNX variants permute [2 1 3]."""
    image = np.asarray(image, dtype=np.float64)
    if image.ndim != 3:
        raise ValueError("Invalid input.")
    if layer_type == "nnet.keras.layer.FlattenCStyleLayer":
        image = np.transpose(image, (2, 1, 0))
    elif layer_type == "nnet.cnn.layer.FlattenLayer":
        pass
    elif layer_type in ("nnet.onnx.layer.FlattenLayer", "nnet.onnx.layer.FlattenInto2dLayer",
                        "nnet.onnx.layer.Flatten3dInto2dLayer"):
        image = np.transpose(image, (1, 0, 2))
    else:
        raise ValueError("Unknown type of flatten layer")
    return image.reshape(1, 1, -1, order="F")


def flatten_reach(I, layer_type):
    """FlattenLayer.reach_single_input, nn/layers/FlattenLayer.m:178-199: evaluate on each of the n+1
    images -> ImageStar 1 x 1 x N x (n+1).  Stars pass through (:218-221)."""
    if isinstance(I, OStar):
        return I
    if not isinstance(I, OImageStar):
        raise TypeError("Invalid input set (ImageStar, ImageZono or VolumeStar)")
    N = I.height * I.width * I.numChannel
    V = np.zeros((1, 1, N, I.numPred + 1))
    for i in range(I.numPred + 1):
        V[0, 0, :, i] = flatten_evaluate(I.V[:, :, :, i], layer_type).reshape(-1)
    return OImageStar(V, I.C, I.d, I.pred_lb, I.pred_ub)


def image_star_affine_map(I: OImageStar, scale, offset) -> OImageStar:
    """ImageStar.affineMap(scale, offset), set/ImageStar.m:431-460: new_V = scale .* V (scalar or
    1x1xC scale broadcast over the image), new_V(:,:,:,1) += offset (scalar, 1x1xC or H x W x C)."""
    V = I.V
    if scale is not None and np.size(scale):
        sc = np.asarray(scale, dtype=np.float64)
        if sc.size != 1 and sc.size != I.numChannel:
            raise ValueError("Inconsistent number of channels between scale array and the ImageStar")
        V = (sc.reshape(-1)[0] if sc.size == 1 else sc.reshape(1, 1, -1, 1)) * V
    else:
        V = V.copy()
    if offset is not None and np.size(offset):
        off = np.asarray(offset, dtype=np.float64)
        if off.size == I.numChannel and off.ndim <= 1:
            off = off.reshape(1, 1, -1)
        V[:, :, :, 0] = V[:, :, :, 0] + off
    return OImageStar(V, I.C, I.d, I.pred_lb, I.pred_ub)


def image_input_evaluate(x, normalization, mean=None, std=None, mn=None, mx=None):
    """ImageInputLayer.evaluate, nn/layers/ImageInputLayer.m:60-117."""
    x = np.asarray(x, dtype=np.float64)
    if normalization == "none":
        return x
    if normalization == "zerocenter":
        return x - np.asarray(mean, dtype=np.float64)
    if normalization == "zscore":
        return (x - np.asarray(mean, dtype=np.float64)) / np.asarray(std, dtype=np.float64).reshape(1, 1, -1)
    if normalization == "rescale-zero-one":
        return (x - mn) / (mx - mn) if mn is not None and mx is not None else x / 255
    if normalization == "rescale-symmetric":
        return 2 * (x - mn) / (mx - mn) - 1 if mn is not None and mx is not None else 2 * x / 255 - 1
    raise ValueError("The normalization method is not supported yet.")


def image_input_reach(I: OImageStar, normalization, mean=None, std=None, mn=None, mx=None) -> OImageStar:
    """ImageInputLayer.reach_star_single_input, nn/layers/ImageInputLayer.m:121-166."""
    if not isinstance(I, OImageStar):
        raise TypeError("Input is not an ImageStar")
    if normalization == "none":
        return I
    if normalization == "zerocenter":
        return image_star_affine_map(I, None, -np.asarray(mean, dtype=np.float64))
    if normalization == "zscore":
        out = image_star_affine_map(I, None, -np.asarray(mean, dtype=np.float64))
        sd = np.asarray(std, dtype=np.float64).reshape(-1)
        for nc in range(out.numChannel):
            out.V[:, :, nc, :] = out.V[:, :, nc, :] / sd[nc]
        return out
    if normalization == "rescale-zero-one":
        if mn is not None and mx is not None:
            out = image_star_affine_map(I, None, -np.asarray(mn, dtype=np.float64))
            out.V = out.V * (1.0 / (mx - mn))
            return out
        return image_star_affine_map(I, 1 / 255, None)
    if normalization == "rescale-symmetric":
        if mn is not None and mx is not None:
            out = image_star_affine_map(I, None, -np.asarray(mn, dtype=np.float64))
            out.V = out.V * (2.0 / (mx - mn))
            return image_star_affine_map(out, None, -1.0)
        return image_star_affine_map(I, 2 / 255, -1.0)
    raise ValueError("The normalization method is not supported yet.")


def layers_reach(I, W, b, f, reach_method, relax_factor=1.0):
    """LayerS.reach, nn/layers/LayerS.m:120-262: affineMap(W, b), then the activation
    ('purelin' and 'softmax' leave the set, 'poslin' -> PosLin.reach)."""
    I1 = affine_map(I, W, b)
    if f in ("purelin", "softmax"):
        return I1
    if f == "poslin":
        return reach_relaxed_star(I1, reach_method, relax_factor)
    raise ValueError("Unsupported activation function, currently support purelin, poslin(ReLU), satlin, satlins, logsig, tansig, softmax")


# --------------------------------------------------------------------------------------
# specification check (the consumer of the reach set)
# --------------------------------------------------------------------------------------
class OHalfSpace:
    """HalfSpace {x | G x <= g}, set/HalfSpace.m:1-33."""

    def __init__(self, G, g):
        G = np.asarray(G, dtype=np.float64)
        if G.ndim == 1:
            G = G.reshape(1, -1)
        g = np.asarray(g, dtype=np.float64)
        if g.ndim == 2 and g.shape[1] != 1:
            raise ValueError("Half-space vector should have one column")
        g = g.reshape(-1)
        if G.shape[0] != g.shape[0]:
            raise ValueError("Inconsistent dimension between half-space matrix and half-space vector")
        self.G = G
        self.g = g
        self.dim = G.shape[1]


def halfspace_contains(H: OHalfSpace, x) -> bool:
    """HalfSpace.contains, set/HalfSpace.m:36-57: no entry of g - G*x is negative."""
    x = np.asarray(x, dtype=np.float64).reshape(-1)
    if x.size != H.dim:
        raise ValueError("Inconsistent dimension between the vector x and the half-space object")
    return not np.any(H.g - H.G @ x < 0)


def is_empty_set(S: OStar) -> bool:
    """Star.isEmptySet, set/Star.m:1216-1232: feasibility LP with a zero objective over
    C*a <= d, predicate_lb <= a <= predicate_ub (utils/lpsolver.m; its box-only shortcut
    :36-50 is restated first).  MATLAB's linprog is replaced by scipy's HiGHS."""
    from scipy.optimize import linprog
    n = S.nVar
    lb = S.predicate_lb if S.predicate_lb is not None and np.size(S.predicate_lb) else None
    ub = S.predicate_ub if S.predicate_ub is not None and np.size(S.predicate_ub) else None
    A, b = S.C, S.d
    if (A.size == 0 or not np.any(A)) and lb is not None and ub is not None \
            and np.all(np.isfinite(lb)) and np.all(np.isfinite(ub)) and (b.size == 0 or np.all(b >= 0)):
        return False  # lpsolver.m:36-50: closed-form optimum over the box, exit flag "l1"
    bounds = [(None if lb is None else lb[i], None if ub is None else ub[i]) for i in range(n)]
    res = linprog(np.zeros(n), A_ub=A if A.size else None, b_ub=b if A.size else None, bounds=bounds, method="highs")
    if res.status == 0:
        return False
    if res.status == 2:
        return True
    raise RuntimeError("LP solver error, status %d: %s" % (res.status, res.message))


def intersect_half_space(S: OStar, H, g):
    """Star.intersectHalfSpace, set/Star.m:555-589: appends C1 = H*V(:,2:end),
    d1 = g - H*V(:,1); returns None when the result is empty."""
    H = np.asarray(H, dtype=np.float64)
    if H.ndim == 1:
        H = H.reshape(1, -1)
    g = np.asarray(g, dtype=np.float64)
    if g.ndim == 2 and g.shape[1] != 1:
        raise ValueError("Halfspace vector should have one column")
    g = g.reshape(-1)
    if H.shape[0] != g.shape[0]:
        raise ValueError("Inconsistent dimension between Halfspace matrix and halfspace vector")
    if H.shape[1] != S.dim:
        raise ValueError("Inconsistent dimension between halfspace and star set")
    C1 = H @ S.V[:, 1:]
    d1 = g - H @ S.V[:, 0]
    out = OStar(S.V, np.vstack([S.C, C1]), np.concatenate([S.d, d1]), S.predicate_lb, S.predicate_ub)
    return None if is_empty_set(out) else out


def verify_specification(reach_set, halfspaces) -> int:
    """utils/verify_specification.m:36-80.  reach_set: a set or a list of sets; halfspaces: one
    OHalfSpace or a list (an OR of unsafe regions).  1 = no set meets any half-space (property
    holds), 2 = some intersection is non-empty (unknown for an over-approximation)."""
    R = reach_set if isinstance(reach_set, (list, tuple)) else [reach_set]
    prop = halfspaces if isinstance(halfspaces, (list, tuple)) else [halfspaces]
    result = 1
    for H in prop:
        for S in R:
            if isinstance(S, OImageStar):
                S = S.to_star()
            if intersect_half_space(S, H.G, H.g) is not None:
                return 2
    return result


def robustness_set(out_size: int, target: int, class_type: str = "max"):
    """NN.robustness_set, nn/NN.m:1334-1368 (target is 0-based here): one single-row half-space
    per other class; for 'max' the row is x_target - x_j <= 0 written as [-e_j + e_target]."""
    if target >= out_size:
        raise ValueError("Target idx must be less than or equal to the output size of the NN.")
    G = np.eye(out_size)
    G = np.delete(G, target, axis=0)
    if class_type == "max":
        G = -G
        G[:, target] = 1.0
    elif class_type == "min":
        G[:, target] = -1.0
    return [OHalfSpace(G[i:i + 1, :], np.zeros(1)) for i in range(G.shape[0])]


def verify_robustness(layers, input_set, reach_method, target, relax_factor=1.0) -> int:
    """NN.verify_robustness -> checkRobust, nn/NN.m:590-640: reach, then the specification check
    against robustness_set(target, 'max') (or the given half-spaces).  An over-approximate method
    never turns 2 into 0."""
    out = nn_reach(layers, input_set, reach_method, relax_factor)
    if isinstance(target, (int, np.integer)):
        layer = [L for L in layers if L["type"] == "fc"][-1]
        target = robustness_set(layer["W"].shape[0], int(target), "max")
    return verify_specification(out, target)

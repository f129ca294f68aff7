"""A hand-built star for the relaxFactor < 1 bookkeeping of the six relax-star heuristics
(nn/funcs/PosLin.m:929-976, 1049-1096, 1167-1256, 1326-1421, 1488-1532, 1604-1645).

Two predicates a1, a2 in [-1, 1] with the one constraint a1 + a2 <= 0: the feasible region is the triangle
with corners (-1,-1), (1,-1), (-1,1), so every LP optimum is the best of three corner values and can be
written down by hand.  All numbers are dyadic, so estimates, sort keys and their ties are exact.

 neuron (1-based)   x = c + g1*a1 + g2*a2        estimateRanges     LP range (over the triangle)
   1                1    + a1   + a2             [-1,    3   ]      [-1,    1   ]
   2               -0.5  + 2a1  + 2a2            [-4.5,  3.5 ]      [-4.5, -0.5 ]   LP shows it inactive
   3                2.5  - 2a1  - 2a2            [-1.5,  6.5 ]      [ 2.5,  6.5 ]   LP shows it active
   4               -2    + 0.5a1                 [-2.5, -1.5 ]      inactive by estimate (map1)
   5                2           + 0.5a2          [ 1.5,  2.5 ]      active by estimate
   6                0.25 + 2a1                   [-1.75, 2.25]      the same
   7               -0.125       + a2             [-1.125,0.875]     the same
   8                0.25 + 0.5a1 + 0.5a2         [-0.75, 1.25]      [-0.75, 0.25]

 map1 = [4], map2 = [1 2 3 6 7 8]; range keys ub-lb = [4 8 8 4 2 2], area keys 0.5*|ub|*|lb| =
 [1.5 7.875 4.875 1.96875 0.4921875 0.46875]; ub(map2) = [3 3.5 6.5 2.25 0.875 1.25], |lb(map2)| =
 [1 4.5 1.5 1.75 1.125 0.75].

The expectations below were derived by walking the reference's statements with these numbers on paper (the
derivation is in the comments of EXPECTED); they are lists of 1-based neuron numbers as MATLAB would hold them.
"""
import numpy as np

V = np.array([
    [1.0, 1.0, 1.0],
    [-0.5, 2.0, 2.0],
    [2.5, -2.0, -2.0],
    [-2.0, 0.5, 0.0],
    [2.0, 0.0, 0.5],
    [0.25, 2.0, 0.0],
    [-0.125, 0.0, 1.0],
    [0.25, 0.5, 0.5],
])
C = np.array([[1.0, 1.0]])
d = np.array([0.0])
PRED_LB = np.array([-1.0, -1.0])
PRED_UB = np.array([1.0, 1.0])

# randperm(6, n1) of the 'random' heuristic, fixed for the test (1-based positions in map2)
RANDPERM = {3: [5, 2, 3]}

# (method, relaxFactor) -> (rows reset [map11], new-predicate neuron order, their lb, their ub)
EXPECTED = {
    # n1 = round(0.5*6) = 3.  Stable descending sort of [4 8 8 4 2 2] -> midx = [2 3 1 4 5 6]:
    # map21 = [2 3 1], map22 = [6 7 8].  xmax = [-0.5 6.5 1] -> map4 = [2], map11 = [4 2]; map6 = [3 1],
    # xmin = [2.5 -1] -> map8 = [1] (lb -1, ub 1).  map9 = [map22; map8].  Neuron 3 is left alone.
    ("relax-star-range", 0.5): ([4, 2], [6, 7, 8, 1], [-1.75, -1.125, -0.75, -1.0], [2.25, 0.875, 1.25, 1.0]),
    # areas sorted: 2 (7.875), 3 (4.875), 6 (1.96875), 1, 7, 8 -> map21 = [2 3 6], map22 = [1 7 8].
    # xmax = [-0.5 6.5 2.25] -> map4 = [2]; map6 = [3 6], xmin = [2.5 -1.75] -> map8 = [6].
    ("relax-star-area", 0.5): ([4, 2], [1, 7, 8, 6], [-1.0, -1.125, -0.75, -1.75], [3.0, 0.875, 1.25, 2.25]),
    # map21 = map2(1:3) = [1 2 3], map22 = [6 7 8]; xmax = [1 -0.5 6.5] -> map4 = [2]; map6 = [1 3],
    # xmin = [-1 2.5] -> map8 = [1].
    ("relax-star-static", 0.5): ([4, 2], [6, 7, 8, 1], [-1.75, -1.125, -0.75, -1.0], [2.25, 0.875, 1.25, 1.0]),
    # midx = [5 2 3] -> map21 = [7 2 3], map22 = setdiff(map2, map21, 'stable') = [1 6 8];
    # xmax = [0.875 -0.5 6.5] -> map4 = [2]; map6 = [7 3], xmin = [-1.125 2.5] -> map8 = [7].
    ("relax-star-random", 0.5): ([4, 2], [1, 6, 8, 7], [-1.0, -1.75, -0.75, -1.125], [3.0, 2.25, 1.25, 0.875]),
    # lu = [3 3.5 6.5 2.25 0.875 1.25 | 1 4.5 1.5 1.75 1.125 0.75]; descending positions
    # [3 8 2 1 4 10 9 6 11 7 5 12]; first 2*n1 = 6: [3 8 2 1 4 10] -> ub_idx = [3 2 1 4], lb_idx = [2 4]:
    # map21 = [3 2 1 6], map22 = [2 6].  xmax = [6.5 -0.5 1 2.25] -> map4 = [2], map6 = [3 1 6], map11 = [4 2].
    # map23 = setdiff([2 6], [2]) = [6], xmin = -1.75 -> map8 = [6], map10 = [].  map24 = setdiff(map2, [2]) =
    # [1 3 6 7 8]; ub(3) = 6.5, ub(1) = 1, ub(6) = 2.25, lb(6) = -1.75; neuron 3 keeps its estimated lb -1.5.
    ("relax-star-bound", 0.5): ([4, 2], [1, 3, 6, 7, 8], [-1.0, -1.5, -1.75, -1.125, -0.75], [1.0, 6.5, 2.25, 0.875, 1.25]),
    # n1 = round(0.75*6) = round(4.5) = 5; first 10 positions [3 8 2 1 4 10 9 6 11 7] -> ub_idx = [3 2 1 4 6],
    # lb_idx = [2 4 3 5 1]: map21 = [3 2 1 6 8], map22 = [2 6 3 7 1].  xmax = [6.5 -0.5 1 2.25 0.25] -> map4 = [2].
    # map23 = [6 3 7 1], xmin = [-1.75 2.5 -1.125 -1] -> map8 = [6 7 1], map10 = [3].  map24 = [1 3 6 7 8] minus
    # [3] = [1 6 7 8]; ub(1) = 1, ub(6) = 2.25, ub(8) = 0.25 (ub(7) not optimised).
    ("relax-star-bound", 0.25): ([4, 2], [1, 6, 7, 8], [-1.0, -1.75, -1.125, -0.75], [1.0, 2.25, 0.875, 0.25]),
    # 2*n1 = 6 <= N = 6: every upper bound is optimised, sorted by ub: map21 = [3 2 1 6 8 7], map22 = [].
    # xmax = [6.5 -0.5 1 2.25 0.25 0.875] -> map4 = [2]; no lower bound is optimised; map24 = [1 3 6 7 8].
    ("relax-star-ub", 0.5): ([4, 2], [1, 3, 6, 7, 8], [-1.0, -1.5, -1.75, -1.125, -0.75], [1.0, 6.5, 2.25, 0.875, 0.25]),
    # n1 = 5, 2*n1 - N = 4 lower bounds by |lb| descending: positions [2 4 3 5] -> map22 = [2 6 3 7];
    # map23 = [6 3 7], xmin = [-1.75 2.5 -1.125] -> map10 = [3]; map24 = [1 6 7 8].
    ("relax-star-ub", 0.25): ([4, 2], [1, 6, 7, 8], [-1.0, -1.75, -1.125, -0.75], [1.0, 2.25, 0.875, 0.25]),
}


class FixedPermutation:
    """Stands in for the random generator of the 'random' heuristic: permutation(n) starts with RANDPERM."""

    def __init__(self, head_1based):
        self.head = [h - 1 for h in head_1based]

    def permutation(self, n):
        rest = [i for i in range(n) if i not in self.head]
        return np.array(self.head + rest)

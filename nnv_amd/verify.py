"""Specification check on device-resident reach sets (utils/verify_specification.m:36-80).

The reference intersects every output set with every half-space of the unsafe region
(Star.intersectHalfSpace, set/Star.m:555-589) and solves one feasibility LP over the dense (C, d)
per pair (Star.isEmptySet, set/Star.m:1216-1232).  Here the device first bounds G*x over the
predicate box for all (set, half-space) pairs in one pass (nnvhip_halfspace_check); only the pairs
that pass leaves undecided go to the LP, for which C and d are materialised lazily, once per set.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import HS_DISJOINT, HS_INSIDE, HS_UNDECIDED, check, f64, ptr
from .sets import ImageStar, SetArray, Star


class HalfSpace:
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

    def contains(self, x) -> bool:
        """HalfSpace.contains, set/HalfSpace.m:36-57."""
        x = np.asarray(x, dtype=np.float64)
        if x.ndim == 2 and x.shape[1] != 1:
            raise ValueError("Input vector x should have one column")
        x = x.reshape(-1)
        if x.size != self.dim:
            raise ValueError("Inconsistent dimension between the vector x and the half-space object")
        return not np.any(self.g - self.G @ x < 0)


class SpecStats:
    """What the last verify_specification call did: pairs decided on the device and LPs solved."""

    def __init__(self):
        self.pairs = 0
        self.disjoint = 0
        self.inside = 0
        self.undecided = 0
        self.lp_solved = 0


last_stats = SpecStats()


def _as_star_handles(reachSet):
    sets = list(reachSet) if isinstance(reachSet, (list, tuple, SetArray)) else [reachSet]
    out = []
    for S in sets:
        if isinstance(S, ImageStar):
            S = S.toStar()
        if not isinstance(S, Star):
            raise TypeError("reach set must be a Star or an ImageStar")
        out.append(S)
    return out


def halfspace_check(sets, halfspaces):
    """Device pass: (verdict[count x n_hs], lo[R x count], hi[R x count]) for stacked half-spaces."""
    sets = _as_star_handles(sets)
    ctx = sets[0].ctx
    N = sets[0].dim
    rows = [0]
    for H in halfspaces:
        if H.dim != N:
            raise ValueError("Inconsistent dimension between halfspace and star set")
        rows.append(rows[-1] + H.G.shape[0])
    G = f64(np.vstack([H.G for H in halfspaces]))
    g = f64(np.concatenate([H.g for H in halfspaces]))
    R, count, n_hs = rows[-1], len(sets), len(halfspaces)
    row_ptr = np.asarray(rows, dtype=np.int64)
    verdict = np.empty((count, n_hs), dtype=np.int32, order="F")
    lo = np.empty((R, count), order="F")
    hi = np.empty((R, count), order="F")
    arr = (C.c_void_p * count)(*[S._h.h for S in sets])
    check(ctx.lib.nnvhip_halfspace_check(ctx.handle, count, arr, n_hs, ptr(row_ptr), ptr(G), ptr(g), N,
                                         ptr(verdict), ptr(lo), ptr(hi)))
    return verdict, lo, hi


def _lp_is_empty(Cm, d, plb, pub) -> bool:
    """Star.isEmptySet's LP (set/Star.m:1222-1230): zero objective over C a <= d and the predicate
    bounds; scipy's HiGHS stands where the reference calls linprog."""
    from scipy.optimize import linprog
    n = Cm.shape[1]
    res = linprog(np.zeros(n), A_ub=Cm, b_ub=d, bounds=np.column_stack([plb, pub]), method="highs")
    if res.status == 0:
        return False
    if res.status == 2:
        return True
    raise RuntimeError("LP solver error, status %d: %s" % (res.status, res.message))


def intersection_is_empty(S: Star, H: HalfSpace, cache=None) -> bool:
    """isempty(S.intersectHalfSpace(H.G, H.g)) by the reference's own LP (set/Star.m:555-589)."""
    ctx = S.ctx
    if cache is not None and "C" in cache:
        Cm, d, plb, pub = cache["C"], cache["d"], cache["plb"], cache["pub"]
    else:
        Cm, d = S.C, S.d
        plb, pub = S.predicate_lb, S.predicate_ub
        if cache is not None:
            cache.update(C=Cm, d=d, plb=plb, pub=pub)
    R, n = H.G.shape[0], S.nVar
    C1 = np.empty((R, n), order="F")
    d1 = np.empty(R)
    check(ctx.lib.nnvhip_halfspace_rows(ctx.handle, S._h.h, R, ptr(f64(H.G)), ptr(f64(H.g)), S.dim, ptr(C1), ptr(d1)))
    last_stats.lp_solved += 1
    return _lp_is_empty(np.vstack([Cm, C1]), np.concatenate([d, d1]), plb, pub)


def _may_be_empty(S) -> bool:
    """True for a set that carries constraint rows of the caller's (it may be empty); False for Star(lb, ub) and
    whatever the layers of this library made of it."""
    flag = C.c_int32(0)
    check(S.ctx.lib.nnvhip_star_has_user_constraints(S._h.h, C.byref(flag)))
    return bool(flag.value)


def verify_specification(reachSet, property, assume_nonempty=None) -> int:
    """utils/verify_specification.m:36-80.  property: a HalfSpace or a list of them (an OR of unsafe
    regions).  Returns 1 when no output set meets any half-space, else 2.

    assume_nonempty: sets produced by reach from a non-empty input set are non-empty (they contain
    the image of every input point), so a pair the device reports INSIDE is a non-empty
    intersection without an LP.  Default (None): decided per set -- a set that goes back to a
    Star(V, C, d, ...) with constraint rows of the caller's may be empty and gets its LP; True / False
    force the choice for every set.
    """
    global last_stats
    last_stats = SpecStats()
    props = list(property) if isinstance(property, (list, tuple)) else [property]
    sets = _as_star_handles(reachSet)
    verdict, _, _ = halfspace_check(sets, props)
    last_stats.pairs = verdict.size
    last_stats.disjoint = int(np.sum(verdict == HS_DISJOINT))
    last_stats.inside = int(np.sum(verdict == HS_INSIDE))
    last_stats.undecided = int(np.sum(verdict == HS_UNDECIDED))
    caches = [dict() for _ in sets]
    # same visiting order as the reference: half-spaces outer, sets inner; first hit returns 2
    for h, H in enumerate(props):
        for k, S in enumerate(sets):
            v = verdict[k, h]
            if v == HS_DISJOINT:
                continue
            if v == HS_INSIDE and (assume_nonempty if assume_nonempty is not None else not _may_be_empty(S)):
                return 2
            if not intersection_is_empty(S, H, caches[k]):
                return 2
    return 1

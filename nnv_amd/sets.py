"""Star / ImageStar / Box: NNV's set classes with the generator matrix resident in HBM.

The classes mirror the fields and methods of the reference that the relax-star reach path and its
callers touch (code/nnv/engine/set/Star.m:13-24, set/ImageStar.m:47-94, set/Box.m).  A set holds an
opaque device handle; property reads (``V``, ``C``, ``d``, ``predicate_lb`` ...) fetch dense arrays
in MATLAB layout on demand.  Index vectors returned to Python are 0-based.
"""
from __future__ import annotations

import collections.abc
import ctypes as C

import numpy as np

from . import _lib
from ._lib import check, f64, ptr


class _Handle:
    """Owns one reference of a device set handle."""

    __slots__ = ("h", "ctx", "_cache")

    def __init__(self, h, ctx):
        self.h = h          # plain integer address (what a c_void_p argument takes) or a c_void_p
        self.ctx = ctx
        self._cache = None  # (N, n, p) once asked for

    def __del__(self):
        try:
            if self.h:
                self.ctx.release_set(self.h)
                self.h = None
        except Exception:
            pass

    def dims(self):
        if self._cache is None:
            N, n, p = C.c_int64(), C.c_int64(), C.c_int64()
            check(self.ctx.lib.nnvhip_star_dims(self.h, C.byref(N), C.byref(n), C.byref(p)))
            self._cache = (N.value, n.value, p.value)
        return self._cache

    def fetch_V(self):
        N, n, _ = self.dims()
        V = np.empty((N, n + 1), dtype=np.float64, order="F")
        check(self.ctx.lib.nnvhip_star_fetch_V(self.h, ptr(V)))
        return V

    def fetch_pred(self):
        _, n, _ = self.dims()
        lb = np.empty(n)
        ub = np.empty(n)
        check(self.ctx.lib.nnvhip_star_fetch_pred_bounds(self.h, ptr(lb), ptr(ub)))
        return lb, ub

    def fetch_constraints(self):
        _, n, p = self.dims()
        Cm = np.empty((p, n), dtype=np.float64, order="F")
        d = np.empty(p)
        check(self.ctx.lib.nnvhip_star_fetch_constraints(self.h, ptr(Cm), ptr(d)))
        return Cm, d

    def fetch_rows(self, rows):
        """V(rows, :) as an R x (n+1) array; rows 0-based."""
        rows = np.ascontiguousarray(np.asarray(rows).reshape(-1), dtype=np.int32)
        _, n, _ = self.dims()
        out = np.empty((rows.size, n + 1), dtype=np.float64, order="F")
        check(self.ctx.lib.nnvhip_star_fetch_rows(self.h, rows.size, ptr(rows), ptr(out)))
        return out

    def ranges(self):
        N, _, _ = self.dims()
        lb = np.empty(N)
        ub = np.empty(N)
        check(self.ctx.lib.nnvhip_estimate_ranges(self.ctx.handle, self.h, ptr(lb), ptr(ub)))
        return lb, ub

    def relu_info(self):
        ni, nc = C.c_int64(), C.c_int64()
        check(self.ctx.lib.nnvhip_star_relu_counts(self.h, C.byref(ni), C.byref(nc)))
        m = nc.value
        idx = np.empty(m, dtype=np.int32)
        lb = np.empty(m)
        ub = np.empty(m)
        check(self.ctx.lib.nnvhip_star_fetch_crossing(self.h, ptr(idx), ptr(lb), ptr(ub)))
        return ni.value, idx, lb, ub


def _make_handles(ctx, raw):
    return [_Handle(C.c_void_p(h), ctx) for h in raw]


def _change_precision(obj, precision):
    """changeVarsPrecision (set/Star.m:1539-1560, set/ImageStar.m): the device store is fp64 only."""
    if precision == "double":
        return obj
    if precision == "single":
        raise ValueError("this library keeps sets in double precision only")
    raise ValueError("Only single or double precision arrays allowed. GpuArray/dlarray are coming.")


def _change_device(obj, deviceTarget):
    """changeDevice (set/Star.m:1563-1585): the set lives in HBM either way; property reads hand out
    host arrays, so both targets return the set itself."""
    if deviceTarget in ("cpu", "gpu"):
        return obj
    raise ValueError("Device target must be 'cpu' or 'gpu'.")


class Box:
    """set/Box.m: hyper-rectangle with centre/generator form and uniform partitioning."""

    def __init__(self, lb, ub):
        lb = np.asarray(lb, dtype=np.float64)
        ub = np.asarray(ub, dtype=np.float64)
        if (lb.ndim == 2 and lb.shape[1] != 1) or (ub.ndim == 2 and ub.shape[1] != 1):
            raise ValueError("lb and ub should be a vector")
        lb = lb.reshape(-1)
        ub = ub.reshape(-1)
        if lb.size != ub.size:
            raise ValueError("Inconsistent dimensions between lb and ub")
        self.lb = lb
        self.ub = ub
        self.dim = lb.size
        self.center = 0.5 * (lb + ub)            # Box.m:35
        self._generators = None

    @property
    def generators(self):
        """dim x (number of non-degenerate dimensions), built on first use: Star(lb, ub) makes the same
        matrix on the device and a partition makes thousands of boxes that never show theirs."""
        if self._generators is None:
            vec = 0.5 * (self.ub - self.lb)      # Box.m:36
            if vec.size > 1:
                keep = np.flatnonzero(vec != 0)  # Box.m:41-43: all-zero columns of diag(vec) are dropped
                gens = np.zeros((vec.size, keep.size))
                gens[keep, np.arange(keep.size)] = vec[keep]
            else:
                gens = np.diag(vec)
            self._generators = gens
        return self._generators

    def singlePartition(self, part_id, part_num):
        """Box.m:61-91; part_id is 0-based."""
        if part_id < 0 or part_id >= self.dim:
            raise ValueError("Invalid partition index")
        if part_num < 1:
            raise ValueError("Invalid partition number")
        if part_num == 1:
            return [self]
        delta = (self.ub[part_id] - self.lb[part_id]) / part_num
        out = []
        for i in range(1, part_num + 1):
            new_lb = self.lb.copy()
            new_ub = self.ub.copy()
            new_lb[part_id] = self.lb[part_id] + (i - 1) * delta
            new_ub[part_id] = new_lb[part_id] + delta
            out.append(Box(new_lb, new_ub))
        return out

    def partition(self, part_indexes, part_numbers):
        """Box.m:96-139: first listed index varies slowest."""
        part_indexes = list(part_indexes)
        part_numbers = list(part_numbers)
        if len(part_indexes) != len(part_numbers):
            raise ValueError("Inconsistent between part_indexes and part_number array, should have the same number of elements")
        for i, (ix, num) in enumerate(zip(part_indexes, part_numbers)):
            if ix < 0 or ix >= self.dim:
                raise ValueError("The %d^th index in part_indexes array is invalid" % (i + 1))
            if num < 1:
                raise ValueError("The %d^th number in part_numbers array is invalid" % (i + 1))
        boxes = [self]
        for ix, num in zip(part_indexes, part_numbers):
            nxt = []
            for b in boxes:
                nxt.extend(b.singlePartition(ix, num))
            boxes = nxt
        return boxes

    def partition_bounds(self, part_indexes, part_numbers):
        """The boxes of partition() as two dim x count matrices (column j = box j), without building
        the Box objects: same arithmetic, statement by statement (Box.m:79-88, 126-137)."""
        part_indexes = list(part_indexes)
        part_numbers = list(part_numbers)
        if len(part_indexes) != len(part_numbers):
            raise ValueError("Inconsistent between part_indexes and part_number array, should have the same number of elements")
        for i, (ix, num) in enumerate(zip(part_indexes, part_numbers)):
            if ix < 0 or ix >= self.dim:
                raise ValueError("The %d^th index in part_indexes array is invalid" % (i + 1))
            if num < 1:
                raise ValueError("The %d^th number in part_numbers array is invalid" % (i + 1))
        # one box per row while they are made; the transposed views returned are column-major dim x count,
        # the layout the device constructor takes (a box is a contiguous column)
        lbs = self.lb.reshape(1, -1).copy()
        ubs = self.ub.reshape(1, -1).copy()
        for ix, num in zip(part_indexes, part_numbers):
            if num == 1:
                continue
            delta = (ubs[:, ix] - lbs[:, ix]) / num                        # one delta per current box
            i = np.arange(1, num + 1, dtype=np.float64)
            new_lb = lbs[:, ix, None] + (i[None, :] - 1) * delta[:, None]  # box-major, part-minor
            new_ub = new_lb + delta[:, None]
            lbs = np.repeat(lbs, num, axis=0)
            ubs = np.repeat(ubs, num, axis=0)
            lbs[:, ix] = new_lb.reshape(-1)
            ubs[:, ix] = new_ub.reshape(-1)
        return lbs.T, ubs.T

    def toStar(self, ctx=None):
        return Star(self.lb, self.ub, ctx=ctx)


class Zono:
    """Zono(c, V), set/Zono.m:13-45: x = c + V*a, -1 <= a <= 1 (a plain host object)."""

    def __init__(self, c, V):
        self.c = np.asarray(c, dtype=np.float64).reshape(-1)
        self.V = np.asarray(V, dtype=np.float64).reshape(self.c.size, -1)
        self.dim = self.c.size

    def affineMap(self, W, b=None):
        """Zono.affineMap, set/Zono.m:47-74."""
        W = np.asarray(W, dtype=np.float64)
        c = W @ self.c
        if b is not None and np.size(b):
            c = c + np.asarray(b, dtype=np.float64).reshape(-1)
        return Zono(c, W @ self.V)


class Star:
    """Device-resident Star: x = c + V*a, C*a <= d, predicate_lb <= a <= predicate_ub.

    Constructors (set/Star.m:29-275): ``Star(V, C, d, pred_lb, pred_ub)``, ``Star(V, C, d)``,
    ``Star(lb, ub)``.  The outer zonotope ``Z`` of the reference (set by Star(lb, ub), mapped along by
    affineMap, dropped by the ReLU step) is not stored: where it exists it is Zono(V(:,1), V(:,2:end)) of the
    same set, and the ``Z`` property builds it from there.
    """

    # defaults of the fields a constructor may leave alone (instances made by _from_handle set only _h)
    state_lb = None
    state_ub = None
    _no_Z = False      # a Star made by ImageStar.toStar (7-argument constructor: no Z, set/ImageStar.m:584-590)
    Z = None
    _lp = None
    _unbounded_predicates = False

    @classmethod
    def _from_handle(cls, handle):
        """A Star around an existing device handle (the layers wrap whole arrays of outputs this way)."""
        s = cls.__new__(cls)
        s._h = handle
        return s

    def __init__(self, *args, ctx=None, _handle=None):
        if _handle is not None:
            self._h = _handle
            return
        ctx = ctx or _lib.default_context()
        lib = ctx.lib
        if len(args) == 2:
            lb = np.asarray(args[0], dtype=np.float64)
            ub = np.asarray(args[1], dtype=np.float64)
            b = Box(lb, ub)  # size checks
            out = (C.c_void_p * 1)()
            check(lib.nnvhip_star_from_box(ctx.handle, b.dim, 1, ptr(f64(b.lb)), ptr(f64(b.ub)), out))
            self._h = _Handle(C.c_void_p(out[0]), ctx)
            self.state_lb = b.lb.copy()
            self.state_ub = b.ub.copy()
            return
        if len(args) in (3, 5):
            V = f64(args[0])
            Cm = np.asarray(args[1], dtype=np.float64)
            d = np.asarray(args[2], dtype=np.float64)
            if V.ndim != 2:
                raise ValueError("Inconsistency between basic matrix and constraint matrix")
            if Cm.ndim == 1:
                Cm = Cm.reshape(1, -1)
            if d.ndim == 2 and d.shape[1] != 1:
                raise ValueError("constraint vector should have one column")
            d = d.reshape(-1)
            if V.shape[1] != Cm.shape[1] + 1:
                raise ValueError("Inconsistency between basic matrix and constraint matrix")
            if Cm.shape[0] != d.shape[0]:
                raise ValueError("Inconsistency between constraint matrix and constraint vector")
            plb = pub = None
            if len(args) == 5 and args[3] is not None and args[4] is not None and np.size(args[3]) and np.size(args[4]):
                plb = np.asarray(args[3], dtype=np.float64)
                pub = np.asarray(args[4], dtype=np.float64)
                if (plb.ndim == 2 and plb.shape[1] != 1) or (pub.ndim == 2 and pub.shape[1] != 1):
                    raise ValueError("predicate lower- or upper-bounds vector should have one column")
                plb = f64(plb.reshape(-1))
                pub = f64(pub.reshape(-1))
                if plb.size != pub.size or plb.size != Cm.shape[1]:
                    raise ValueError("Inconsistency between number of predicate variables and predicate lower- or upper-bounds vector")
            Cm = f64(Cm)
            d = f64(d)
            out = C.c_void_p()
            check(lib.nnvhip_star_create(ctx.handle, V.shape[0], Cm.shape[1], ptr(V), ptr(plb), ptr(pub),
                                         ptr(Cm) if Cm.size else None, ptr(d) if d.size else None, Cm.shape[0],
                                         C.byref(out)))
            self._h = _Handle(out, ctx)
            # no bounds given: the device uses estimateRanges' default [-1, 1] (set/Star.m:1091-1096), the LP
            # methods leave the predicates free as the reference's empty predicate_lb/ub do
            self._unbounded_predicates = plb is None
            return
        raise ValueError("Invalid number of input arguments (should be 0, 1, 2, 3, 5, 6 or 7)")

    # ---- array construction --------------------------------------------------------------
    @staticmethod
    def from_boxes(lbs, ubs, ctx=None):
        """Array of Star(lb, ub) for the columns of two N x count matrices, built in one device
        arena (the Star array NN.reach accepts, nn/NN.m:204-207)."""
        ctx = ctx or _lib.default_context()
        lbs = f64(lbs)
        ubs = f64(ubs)
        if lbs.shape != ubs.shape or lbs.ndim != 2:
            raise ValueError("Inconsistent dimensions between lb and ub")
        N, count = lbs.shape
        out = (C.c_void_p * count)()
        check(ctx.lib.nnvhip_star_from_box(ctx.handle, N, count, ptr(lbs), ptr(ubs), out))
        # state_lb / state_ub of the elements (set/Star.m:232-233) are columns of private copies
        return SetArray(ctx, out, state=(lbs.copy(order="F"), ubs.copy(order="F")))

    # ---- NNV properties ------------------------------------------------------------------
    @property
    def ctx(self):
        return self._h.ctx

    @property
    def dim(self):
        return self._h.dims()[0]

    @property
    def nVar(self):
        return self._h.dims()[1]

    @property
    def V(self):
        return self._h.fetch_V()

    @property
    def C(self):
        return self._h.fetch_constraints()[0]

    @property
    def d(self):
        return self._h.fetch_constraints()[1]

    @property
    def predicate_lb(self):
        return self._h.fetch_pred()[0]

    @property
    def predicate_ub(self):
        return self._h.fetch_pred()[1]

    @property
    def Z(self):
        """The outer zonotope the reference's Star holds here (set/Star.m:230-236, 332-340), or None."""
        if self._no_Z:
            return None
        flag = C.c_int32(0)
        check(self.ctx.lib.nnvhip_star_has_zono(self._h.h, C.byref(flag)))
        if not flag.value:
            return None
        V = self._h.fetch_V()
        return Zono(V[:, 0].copy(), V[:, 1:].copy())

    # ---- methods on the path -------------------------------------------------------------
    def affineMap(self, W, b=None):
        """Star.affineMap, set/Star.m:313-343."""
        from .layers import FullyConnectedLayer
        W = np.asarray(W, dtype=np.float64)
        if W.ndim != 2 or W.shape[1] != self.dim:
            raise ValueError("Inconsistency between the affine mapping matrix and dimension of the star set")
        if b is not None and np.size(b):
            b = np.asarray(b, dtype=np.float64)
            if b.ndim == 2 and b.shape[1] != 1:
                raise ValueError("Mapping vector should have one column")
            if b.reshape(-1).shape[0] != W.shape[0]:
                raise ValueError("Inconsistency between the mapping vec and mapping matrix")
        else:
            b = None
        return FullyConnectedLayer._map(self.ctx, W, b, [self])[0]

    def estimateRanges(self):
        """Star.estimateRanges, set/Star.m:1078-1106 -> (lb, ub)."""
        return self._h.ranges()

    # ---- LP-based ranges (host LP fed from the resident set) -------------------------------
    def _lp_problem(self):
        """(C as a sparse matrix, d, predicate bounds) of this set, fetched once."""
        if self._lp is None:
            from scipy import sparse
            Cm, d = self._h.fetch_constraints()
            if self._unbounded_predicates:                        # Star(V, C, d): predicate_lb/ub are []
                bounds = np.column_stack([np.full(self.nVar, -np.inf), np.full(self.nVar, np.inf)])
            else:
                bounds = np.column_stack(self._h.fetch_pred())
            self._lp = (sparse.csr_matrix(Cm), d, bounds)
        return self._lp

    def _lp_min(self, f):
        """min f'a over C a <= d, pred_lb <= a <= pred_ub (lpsolver's call in set/Star.m:773); scipy's
        HiGHS stands where the reference calls linprog / glpk."""
        from scipy.optimize import linprog
        Cs, d, bounds = self._lp_problem()
        if Cs.nnz == 0 and np.all(np.isfinite(bounds)) and (d.size == 0 or np.all(d >= 0)):
            # utils/lpsolver.m:36-50: nothing but the box -> closed form, no solver call
            return float(np.sum(np.minimum(f * bounds[:, 0], f * bounds[:, 1])))
        res = linprog(f, A_ub=Cs if Cs.shape[0] else None, b_ub=d if Cs.shape[0] else None, bounds=bounds, method="highs")
        if res.status != 0:
            raise RuntimeError("Cannot find an optimal solution, exitflag = %d" % res.status)
        return res.fun

    def _extremes(self, index, sign):
        index = np.asarray(index).reshape(-1)
        if index.size and (index.min() < 0 or index.max() >= self.dim):
            raise ValueError("Invalid index")
        out = np.empty(index.size)
        if index.size == 0:
            return out
        rows = self._h.fetch_rows(index)
        for t in range(index.size):
            f = rows[t, 1:]
            if not f.any():
                out[t] = rows[t, 0]          # all(f(:)==0): the centre entry itself
            else:
                out[t] = sign * self._lp_min(sign * f) + rows[t, 0]
        return out

    def getMin(self, index, lp_solver="linprog"):
        """Star.getMin, set/Star.m:744-781 (index 0-based)."""
        return float(self._extremes([index], 1.0)[0])

    def getMax(self, index, lp_solver="linprog"):
        """Star.getMax, set/Star.m:859-895 (index 0-based)."""
        return float(self._extremes([index], -1.0)[0])

    def getMins(self, map, par_option="single", dis_option=None, lp_solver="linprog"):
        """Star.getMins, set/Star.m:784-856: one LP per listed state (0-based list)."""
        if par_option not in (None, "", "single", "parallel") and not (isinstance(par_option, (list, tuple)) and len(par_option) == 0):
            raise ValueError("Unknown parallel option")
        return self._extremes(map, 1.0)

    def getMaxs(self, map, par_option="single", dis_option=None, lp_solver="linprog"):
        """Star.getMaxs, set/Star.m:898-970."""
        if par_option not in (None, "", "single", "parallel") and not (isinstance(par_option, (list, tuple)) and len(par_option) == 0):
            raise ValueError("Unknown parallel option")
        return self._extremes(map, -1.0)

    def getRange(self, index):
        """Star.getRange, set/Star.m:710-741 -> (xmin, xmax)."""
        return self.getMin(index), self.getMax(index)

    def getRanges(self, lp_solver="linprog"):
        """Star.getRanges, set/Star.m:973-990: 2 LPs per state; empty arrays for an empty set."""
        from scipy.optimize import linprog
        Cs, d, bounds = self._lp_problem()
        if Cs.shape[0] and linprog(np.zeros(self.nVar), A_ub=Cs, b_ub=d, bounds=bounds, method="highs").status == 2:
            return np.empty(0), np.empty(0)
        idx = np.arange(self.dim)
        return self._extremes(idx, 1.0), self._extremes(idx, -1.0)

    def toImageStar(self, height, width, numChannel):
        """Star.toImageStar, set/Star.m:1398-1418: a reshape; the device data is shared."""
        if self.dim != height * width * numChannel:
            raise ValueError("Inconsistent dimension in the ImageStar and the original Star set")
        im = ImageStar(_handle=self._h, shape=(height, width, numChannel))
        if self.state_lb is not None and self.state_ub is not None:
            im.im_lb = np.asarray(self.state_lb).reshape((height, width, numChannel), order="F")
            im.im_ub = np.asarray(self.state_ub).reshape((height, width, numChannel), order="F")
        return im

    def relu_info(self):
        """For a set returned by the ReLU step: (n_inactive, crossing index (0-based, new-predicate
        order), lb(crossing), ub(crossing))."""
        return self._h.relu_info()

    def changeVarsPrecision(self, precision):
        return _change_precision(self, precision)

    def changeDevice(self, deviceTarget):
        return _change_device(self, deviceTarget)

    @staticmethod
    def estimateRanges_array(sets):
        """estimateRanges of every set of an array in one device call -> (lb, ub), dim x count each."""
        if not isinstance(sets, SetArray):
            sets = list(sets)
        if not len(sets):
            return np.empty((0, 0)), np.empty((0, 0))
        ctx = sets[0].ctx
        N = sets[0]._h.dims()[0]          # Star or ImageStar: the flattened dimension
        lb = np.empty((N, len(sets)), order="F")
        ub = np.empty((N, len(sets)), order="F")
        arr = sets.handles() if isinstance(sets, SetArray) else (C.c_void_p * len(sets))(*[s._h.h for s in sets])
        check(ctx.lib.nnvhip_estimate_ranges_batch(ctx.handle, len(sets), arr, ptr(lb), ptr(ub)))
        return lb, ub


class ImageStar:
    """Device-resident ImageStar (set/ImageStar.m:47-94): V is H x W x C x (numPred+1).

    Constructors: ``ImageStar(V, C, d, pred_lb, pred_ub)`` (:172-227) and
    ``ImageStar(lb_image, ub_image)`` (:302-343).
    """

    def __init__(self, *args, ctx=None, _handle=None, shape=None):
        self.im_lb = None
        self.im_ub = None
        if _handle is not None:
            self._h = _handle
            self.height, self.width, self.numChannel = shape
            return
        if len(args) == 2:
            lb_im = np.asarray(args[0], dtype=np.float64)
            ub_im = np.asarray(args[1], dtype=np.float64)
            if lb_im.size == 0:
                raise ValueError("Invalid lower bound image")
            if ub_im.size == 0:
                raise ValueError("Invalid upper bound image")
            if lb_im.shape != ub_im.shape:
                raise ValueError("Inconsistency between lower bound image and upper bound image")
            if lb_im.ndim == 2:
                lb_im = lb_im[:, :, None]
                ub_im = ub_im[:, :, None]
            if lb_im.ndim != 3:
                raise ValueError("Inconsistency between lower bound image and upper bound image")
            h, w, c = lb_im.shape
            S = Star(lb_im.reshape(-1, order="F"), ub_im.reshape(-1, order="F"), ctx=ctx)
            self._h = S._h
            self.height, self.width, self.numChannel = h, w, c
            self.im_lb = lb_im
            self.im_ub = ub_im
            return
        if len(args) == 5:
            V = np.asarray(args[0], dtype=np.float64)
            Cm = np.asarray(args[1], dtype=np.float64)
            d = np.asarray(args[2], dtype=np.float64)
            if Cm.ndim == 1:
                Cm = Cm.reshape(1, -1)
            if d.ndim == 2 and d.shape[1] != 1:
                raise ValueError("Invalid constraint vector, vector should have one column")
            if Cm.shape[0] != d.reshape(-1).shape[0]:
                raise ValueError("Inconsistent dimension between constraint matrix and constraint vector")
            plb = np.asarray(args[3], dtype=np.float64).reshape(-1)
            pub = np.asarray(args[4], dtype=np.float64).reshape(-1)
            if Cm.shape[1] != plb.size or Cm.shape[1] != pub.size:
                raise ValueError("Number of predicates is different from the size of the lower bound or upper bound predicate vector")
            if V.ndim == 2:
                V = V[:, :, None, None]
            elif V.ndim == 3:
                V = V[:, :, :, None]
            if V.ndim != 4:
                raise ValueError("Invalid basis matrix")
            if V.shape[3] != Cm.shape[1] + 1:
                raise ValueError("Inconsistency between the basis matrix and the number of predicate variables")
            h, w, c, g = V.shape
            S = Star(V.reshape(h * w * c, g, order="F"), Cm, d, plb, pub, ctx=ctx)
            self._h = S._h
            self.height, self.width, self.numChannel = h, w, c
            return
        raise ValueError("Invalid number of input arguments")

    @property
    def ctx(self):
        return self._h.ctx

    @property
    def numPred(self):
        return self._h.dims()[1]

    @property
    def V(self):
        V = self._h.fetch_V()
        return V.reshape((self.height, self.width, self.numChannel, V.shape[1]), order="F")

    @property
    def C(self):
        return self._h.fetch_constraints()[0]

    @property
    def d(self):
        return self._h.fetch_constraints()[1]

    @property
    def pred_lb(self):
        return self._h.fetch_pred()[0]

    @property
    def pred_ub(self):
        return self._h.fetch_pred()[1]

    def toStar(self):
        """ImageStar.toStar, set/ImageStar.m:569-592: flatten in column-major order (shared data)."""
        S = Star(_handle=self._h)
        S._no_Z = True
        if self.im_lb is not None and self.im_ub is not None:
            S.state_lb = np.asarray(self.im_lb).reshape(-1, order="F")
            S.state_ub = np.asarray(self.im_ub).reshape(-1, order="F")
        return S

    def estimateRanges(self):
        """ImageStar.estimateRanges, set/ImageStar.m:836-885 -> (image_lb, image_ub); cached."""
        if self.im_lb is None or self.im_ub is None:
            lb, ub = self._h.ranges()
            shp = (self.height, self.width, self.numChannel)
            self.im_lb = lb.reshape(shp, order="F")
            self.im_ub = ub.reshape(shp, order="F")
        return self.im_lb, self.im_ub

    def changeVarsPrecision(self, precision):
        return _change_precision(self, precision)

    def changeDevice(self, deviceTarget):
        return _change_device(self, deviceTarget)

    def relu_info(self):
        return self._h.relu_info()


class SetArray(collections.abc.Sequence):
    """The array of sets a layer returns for an array of input sets (the object arrays NN.reach
    hands from layer to layer and keeps in reachSet, nn/NN.m:1544-1547).

    It holds the device handles.  The Star / ImageStar object of an element is made when that element
    is first read, so passing an array of a thousand sets through a network costs no Python work per
    set; indexing, iteration, ``len`` and slicing (a plain list of the elements) behave as for a list.
    """

    __slots__ = ("ctx", "_raw", "_shapes", "_items", "_state")

    def __init__(self, ctx, raw, shapes=None, state=None):
        self.ctx = ctx
        self._raw = raw          # ctypes array of handles; this object owns one reference of each
        self._shapes = shapes    # None: Stars only; else per element None (Star) or (height, width, numChannel)
        self._items = None       # the elements read so far (each then owns its handle's reference)
        self._state = state      # None, or (lb, ub) matrices whose column i is element i's state_lb / state_ub

    def __len__(self):
        return len(self._raw)

    def __getitem__(self, i):
        if isinstance(i, slice):
            return [self[k] for k in range(*i.indices(len(self._raw)))]
        n = len(self._raw)
        if i < 0:
            i += n
        if not 0 <= i < n:
            raise IndexError("set array index out of range")
        if self._items is None:
            self._items = [None] * n
        it = self._items[i]
        if it is None:
            hd = _Handle(self._raw[i], self.ctx)
            shape = None if self._shapes is None else self._shapes[i]
            it = Star._from_handle(hd) if shape is None else ImageStar(_handle=hd, shape=shape)
            if self._state is not None:
                it.state_lb = self._state[0][:, i]
                it.state_ub = self._state[1][:, i]
            self._items[i] = it
        return it

    def __iter__(self):
        for i in range(len(self._raw)):
            yield self[i]

    def handles(self):
        """The handles as the ctypes array a batched entry point takes."""
        return self._raw

    @property
    def shapes(self):
        """None when every element is a Star, else one entry per element: None or the image shape."""
        return self._shapes

    def __repr__(self):
        return "<SetArray of %d sets>" % len(self._raw)

    def __del__(self):
        try:
            raw = self._raw
            if self._items is not None:      # elements that were read keep their handle
                for i, it in enumerate(self._items):
                    if it is not None:
                        raw[i] = None
            self.ctx.release_sets(len(raw), raw)
        except Exception:
            pass

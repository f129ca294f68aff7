"""ctypes binding of libnnvhip.so.  There is no CPU fallback: a missing library is an error."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libnnvhip.so")

OK, ERR_SHAPE, ERR_METHOD, ERR_RELAX_FACTOR, ERR_OOM, ERR_HIP, ERR_ARG = range(7)
ORDER_INDEX, ORDER_AREA, ORDER_RANGE = 0, 1, 2
HS_DISJOINT, HS_UNDECIDED, HS_INSIDE = 1, 2, 3

# every entry point declared in include/nnvhip.h
SYMBOLS = [
    "nnvhip_create", "nnvhip_destroy", "nnvhip_last_error", "nnvhip_synchronize", "nnvhip_set_timing",
    "nnvhip_last_op_time_ms", "nnvhip_set_dense_affine", "nnvhip_set_eager_columns", "nnvhip_set_eager_relu", "nnvhip_set_small_chain", "nnvhip_upload_stats", "nnvhip_kernel_time", "nnvhip_probe_copy_bandwidth",
    "nnvhip_trim_pool", "nnvhip_pool_stats", "nnvhip_star_create",
    "nnvhip_star_from_box", "nnvhip_star_retain", "nnvhip_star_release", "nnvhip_star_release_array", "nnvhip_star_dims", "nnvhip_star_has_user_constraints", "nnvhip_star_has_zono",
    "nnvhip_star_fetch_V", "nnvhip_star_fetch_pred_bounds", "nnvhip_star_fetch_constraints",
    "nnvhip_star_relu_counts", "nnvhip_star_fetch_crossing", "nnvhip_estimate_ranges",
    "nnvhip_estimate_ranges_batch", "nnvhip_fc_create", "nnvhip_fc_destroy", "nnvhip_conv2d_create",
    "nnvhip_conv2d_destroy", "nnvhip_conv2d_output_size", "nnvhip_affine_fc", "nnvhip_affine_conv2d",
    "nnvhip_relu_relax", "nnvhip_halfspace_check", "nnvhip_halfspace_rows", "nnvhip_rowmap_create",
    "nnvhip_rowmap_destroy", "nnvhip_affine_rowmap", "nnvhip_avgpool2d_create", "nnvhip_avgpool2d_destroy",
    "nnvhip_avgpool2d_output_size", "nnvhip_affine_avgpool2d", "nnvhip_permute_rows",
    "nnvhip_star_fetch_rows", "nnvhip_relu_apply_lists", "nnvhip_probe_mfma_peak",
    "nnvhip_estimate_ranges_static", "nnvhip_debug_mailbox_pack", "nnvhip_debug_mailbox_unpack",
    "nnvhip_debug_set_relu_call_number", "nnvhip_reach_layers", "nnvhip_relu_reduce_mem",
    "nnvhip_set_switch", "nnvhip_hint_next_fc", "nnvhip_debug_counters", "nnvhip_debug_relu_bounds", "nnvhip_weight_cache_stats", "nnvhip_weight_cache_release", "nnvhip_debug_weak_weight_hash",
]


# route switches of a context (nnvhip_set_switch) and the environment variable each one starts from
SWITCH_ENV = {"dense_affine": "NNVHIP_DENSE_AFFINE", "eager_rows": "NNVHIP_EAGER_ROWS", "eager_tail": "NNVHIP_EAGER_TAIL",
              "eager_cols": "NNVHIP_EAGER_COLS", "poison_pending": "NNVHIP_POISON_PENDING",
              "no_small_chain": "NNVHIP_NO_SMALL_CHAIN", "no_conv_mask": "NNVHIP_NO_CONV_MASK",
              "no_conv_boxes": "NNVHIP_NO_CONV_BOXES", "no_row_deltas": "NNVHIP_NO_ROW_DELTAS",
              "no_sum_shortcuts": "NNVHIP_NO_SUM_SHORTCUTS"}


class NNVHipError(RuntimeError):
    """A HIP runtime failure or an invalid handle."""


class NNVHipOutOfMemory(MemoryError):
    pass


_lib = None


def load():
    """Load the in-tree HIP library; raises if it has not been built (python -m nnv_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("nnv_amd/libnnvhip.so is missing: build it with `python -m nnv_amd.build` "
                          "(there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    p, i64, dbl = C.c_void_p, C.c_int64, C.c_double
    pp = C.POINTER(C.c_void_p)
    pi64 = C.POINTER(C.c_int64)
    sig = {
        "nnvhip_create": [C.c_int, pp],
        "nnvhip_destroy": [p],
        "nnvhip_synchronize": [p],
        "nnvhip_set_timing": [p, C.c_int],
        "nnvhip_set_dense_affine": [p, C.c_int],
        "nnvhip_set_eager_columns": [p, C.c_int],
        "nnvhip_set_eager_relu": [p, C.c_int],
        "nnvhip_set_small_chain": [p, C.c_int],
        "nnvhip_upload_stats": [p, p, p, p],
        "nnvhip_last_op_time_ms": [p, C.POINTER(dbl)],
        "nnvhip_kernel_time": [p, C.c_int, C.POINTER(dbl), pi64, C.POINTER(dbl), C.c_int],
        "nnvhip_probe_copy_bandwidth": [p, i64, C.c_int, C.POINTER(dbl)],
        "nnvhip_trim_pool": [p],
        "nnvhip_pool_stats": [p, pi64, pi64],
        "nnvhip_star_create": [p, i64, i64, p, p, p, p, p, i64, pp],
        "nnvhip_star_from_box": [p, i64, i64, p, p, pp],
        "nnvhip_star_retain": [p],
        "nnvhip_star_release": [p],
        "nnvhip_star_release_array": [i64, pp],
        "nnvhip_star_dims": [p, pi64, pi64, pi64],
        "nnvhip_star_has_user_constraints": [p, p],
        "nnvhip_star_has_zono": [p, p],
        "nnvhip_star_fetch_V": [p, p],
        "nnvhip_star_fetch_rows": [p, i64, p, p],
        "nnvhip_star_fetch_pred_bounds": [p, p, p],
        "nnvhip_star_fetch_constraints": [p, p, p],
        "nnvhip_star_relu_counts": [p, pi64, pi64],
        "nnvhip_star_fetch_crossing": [p, p, p, p],
        "nnvhip_estimate_ranges": [p, p, p, p],
        "nnvhip_estimate_ranges_batch": [p, i64, pp, p, p],
        "nnvhip_fc_create": [p, p, p, i64, i64, pp],
        "nnvhip_fc_destroy": [p],
        "nnvhip_conv2d_create": [p, p, p, i64, i64, i64, i64, pi64, pi64, pi64, pp],
        "nnvhip_conv2d_destroy": [p],
        "nnvhip_conv2d_output_size": [p, i64, i64, pi64, pi64],
        "nnvhip_affine_fc": [p, p, i64, pp, pp],
        "nnvhip_affine_conv2d": [p, p, i64, i64, i64, pp, pp],
        "nnvhip_relu_relax": [p, C.c_int, dbl, i64, pp, pp],
        "nnvhip_relu_apply_lists": [p, p, i64, p, i64, p, p, p, pp],
        "nnvhip_probe_mfma_peak": [p, C.c_int, C.POINTER(dbl)],
        "nnvhip_halfspace_check": [p, i64, pp, i64, p, p, p, i64, p, p, p],
        "nnvhip_halfspace_rows": [p, p, i64, p, p, i64, p, p],
        "nnvhip_rowmap_create": [p, i64, C.c_int32, p, p, p, pp],
        "nnvhip_rowmap_destroy": [p],
        "nnvhip_affine_rowmap": [p, p, i64, pp, pp],
        "nnvhip_avgpool2d_create": [p, pi64, pi64, pi64, pp],
        "nnvhip_avgpool2d_destroy": [p],
        "nnvhip_avgpool2d_output_size": [p, i64, i64, pi64, pi64],
        "nnvhip_affine_avgpool2d": [p, p, i64, i64, i64, pp, pp],
        "nnvhip_permute_rows": [p, i64, p, i64, pp, pp],
        "nnvhip_estimate_ranges_static": [p, p, p, p],
        "nnvhip_debug_mailbox_pack": [C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_uint64)],
        "nnvhip_debug_mailbox_unpack": [C.c_uint64, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                                        C.POINTER(C.c_int32)],
        "nnvhip_debug_set_relu_call_number": [p, i64],
        "nnvhip_reach_layers": [p, i64, p, p, p, C.c_int, dbl, i64, pp, pp],
        "nnvhip_relu_reduce_mem": [p, p, i64, i64, i64, pp, p, p],
        "nnvhip_set_switch": [p, C.c_char_p, C.c_int],
        "nnvhip_hint_next_fc": [p, p],
        "nnvhip_debug_counters": [p, pi64, pi64, pi64, pi64],
        "nnvhip_debug_relu_bounds": [p, pi64, pi64],
        "nnvhip_weight_cache_stats": [p, pi64, pi64, pi64],
        "nnvhip_weight_cache_release": [p, pi64],
        "nnvhip_debug_weak_weight_hash": [C.c_int],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = C.c_int
    lib.nnvhip_last_error.argtypes = []
    lib.nnvhip_last_error.restype = C.c_char_p
    _lib = lib
    return lib


def check(status: int):
    """Turn a non-zero status into the exception NNV's error() call corresponds to."""
    if status == OK:
        return
    msg = load().nnvhip_last_error().decode("utf-8", "replace")
    if status in (ERR_SHAPE, ERR_METHOD, ERR_RELAX_FACTOR):
        raise ValueError(msg)
    if status == ERR_OOM:
        raise NNVHipOutOfMemory(msg)
    raise NNVHipError(msg)


def f64(a, order="F"):
    """Contiguous column-major fp64 copy/view of a host array (MATLAB memory layout)."""
    return np.require(np.asarray(a, dtype=np.float64), dtype=np.float64, requirements=["F" if order == "F" else "C", "A"])


def ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


_default_ctx = None


class Context:
    """One GPU context: stream, device memory pool, per-layer timer."""

    def __init__(self, device: int = 0):
        lib = load()
        h = C.c_void_p()
        check(lib.nnvhip_create(int(device), C.byref(h)))
        self.handle = h
        self.lib = lib
        self.device = device
        self.release_set = lib.nnvhip_star_release   # looked up once: every set handle calls it when it dies
        self.release_sets = lib.nnvhip_star_release_array
        self.eager_columns = bool(os.environ.get("NNVHIP_EAGER_COLS"))
        # the route switches as the library read them from the environment; set_switch keeps the mirror current
        self.switches = {nm: os.environ.get(env) is not None for nm, env in SWITCH_ENV.items()}

    def switch_is_on(self, *names) -> bool:
        """Whether any of the named route switches is on (the Python side's record of nnvhip_set_switch)."""
        return any(self.switches[nm] for nm in names)

    def synchronize(self):
        check(self.lib.nnvhip_synchronize(self.handle))

    def set_timing(self, level):
        """0/False: off; 1/True: per-layer device times; 2: also per-kernel timers (kernel_time)."""
        check(self.lib.nnvhip_set_timing(self.handle, int(level)))

    def set_eager_columns(self, enabled):
        """True: FC layers write the columns they gather from their weights in the call itself; False
        (default): those columns are written when somebody reads them."""
        check(self.lib.nnvhip_set_eager_columns(self.handle, 1 if enabled else 0))
        self.eager_columns = bool(enabled)
        self.switches["eager_cols"] = bool(enabled)

    def set_eager_relu(self, enabled):
        """True: the ReLU step writes its whole output matrix in the call (reset rows zeroed, appended
        columns stored); False (default): both are recorded on the handle and written on first read."""
        check(self.lib.nnvhip_set_eager_relu(self.handle, 1 if enabled else 0))
        self.switches["eager_rows"] = self.switches["eager_tail"] = bool(enabled)

    def set_small_chain(self, enabled):
        """True (default): NN.reach of a small FC / ReLU network is one launch (nnvhip_reach_layers); False: such
        networks go layer by layer like every other."""
        check(self.lib.nnvhip_set_small_chain(self.handle, 1 if enabled else 0))
        self.switches["no_small_chain"] = not enabled

    def set_dense_affine(self, enabled):
        """True: FC layers run as the full dense contraction; False (default): products with the
        structural zeros recorded on the set handles are left out (same result)."""
        check(self.lib.nnvhip_set_dense_affine(self.handle, 1 if enabled else 0))
        self.switches["dense_affine"] = bool(enabled)

    def last_op_time_ms(self) -> float:
        ms = C.c_double()
        check(self.lib.nnvhip_last_op_time_ms(self.handle, C.byref(ms)))
        return ms.value

    def kernel_time(self, which, reset=True):
        """(total ms, launches, work) of a kernel group accumulated while timing was enabled:
        0 = FC GEMM, 1 = convolution (work = dense flop); 2 = estimateRanges pass, 3 = ReLU apply pass
        (work = algorithmic bytes)."""
        ms, n, fl = C.c_double(), C.c_int64(), C.c_double()
        check(self.lib.nnvhip_kernel_time(self.handle, int(which), C.byref(ms), C.byref(n), C.byref(fl), 1 if reset else 0))
        return ms.value, n.value, fl.value

    def probe_mfma_peak(self, reps=3) -> float:
        """TFLOP/s of a register-resident fp64 MFMA loop on every CU (practical matrix-pipe ceiling)."""
        t = C.c_double()
        check(self.lib.nnvhip_probe_mfma_peak(self.handle, int(reps), C.byref(t)))
        return t.value

    def probe_copy_bandwidth(self, nbytes=1 << 30, reps=5) -> float:
        """Achieved read+write GB/s of a plain copy kernel over nbytes (practical HBM ceiling)."""
        g = C.c_double()
        check(self.lib.nnvhip_probe_copy_bandwidth(self.handle, int(nbytes), int(reps), C.byref(g)))
        return g.value

    def pool_stats(self):
        a, b = C.c_int64(), C.c_int64()
        check(self.lib.nnvhip_pool_stats(self.handle, C.byref(a), C.byref(b)))
        return a.value, b.value

    def upload_stats(self):
        """(layers whose weights were uploaded, bytes of those uploads, all host-to-device bytes) since the
        context was created."""
        a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
        check(self.lib.nnvhip_upload_stats(self.handle, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def trim_pool(self):
        check(self.lib.nnvhip_trim_pool(self.handle))

    def debug_counters(self):
        """{device_mallocs, staging_waits, deferred_handles, live_handles} since the context was created."""
        v = [C.c_int64() for _ in range(4)]
        check(self.lib.nnvhip_debug_counters(self.handle, *[C.byref(x) for x in v]))
        return dict(zip(("device_mallocs", "staging_waits", "deferred_handles", "live_handles"), (x.value for x in v)))

    def relu_bounds_counts(self):
        """(sets whose ReLU step appended its predicate bounds in place, sets whose step copied the old ones)."""
        a, b = C.c_int64(), C.c_int64()
        check(self.lib.nnvhip_debug_relu_bounds(self.handle, C.byref(a), C.byref(b)))
        return a.value, b.value

    def hint_next_fc(self, weights):
        """nnvhip_hint_next_fc: the FC layer (its device weights, or None) that will follow the next ReLU step."""
        check(self.lib.nnvhip_hint_next_fc(self.handle, weights.h if weights is not None else None))

    def set_switch(self, name: str, on: bool):
        """One of the route switches a context otherwise reads from the environment (nnvhip_set_switch)."""
        check(self.lib.nnvhip_set_switch(self.handle, name.encode(), 1 if on else 0))
        self.switches[name] = bool(on)
        if name == "eager_cols":
            self.eager_columns = bool(on)

    def weight_cache_stats(self):
        """(cached layers, their device bytes, device bytes of layers only the cache still references)."""
        a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
        check(self.lib.nnvhip_weight_cache_stats(self.handle, C.byref(a), C.byref(b), C.byref(c)))
        return a.value, b.value, c.value

    def weight_cache_release(self) -> int:
        """Frees the cached layers that no layer object references any more; returns how many went."""
        n = C.c_int64()
        check(self.lib.nnvhip_weight_cache_release(self.handle, C.byref(n)))
        return n.value


def default_context() -> Context:
    global _default_ctx
    if _default_ctx is None:
        _default_ctx = Context(int(os.environ.get("NNVHIP_DEVICE", "0")))
    return _default_ctx

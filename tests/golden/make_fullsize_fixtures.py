"""Writes the full-size fixtures of configurations 4 and 5.

tests/golden/cfg4_fullsize_relax_star_area.npz: what the CPU oracle (oracle/nnv_oracle.py) computes for
configuration 4 (the 32x32x3 CNN) at its full size under relax-star-area, in a form small enough to commit.

The oracle needs about 100 s and several GB for this reach, too much for a test that runs with every GPU check, so
its answers are recorded once:
  * for every ReLU layer the number of inactive neurons and the crossing neurons in new-predicate order (exact
    integers: what BASELINE's "bit-exact classification, crossing-index sets and new-predicate ordering" asks for);
  * for every layer 512 entries of the generator matrix at seeded random positions (row, column) and the matrix's
    shape;
  * the estimated ranges of the output set.
tests/test_gpu_fullsize.py compares the device path with these.

tests/golden/cfg5_fullsize_relax_star_area.npz: configuration 5 (the 1024 sub-boxes of configuration 2's input box on
configuration 2's network), every set reached on its own by the oracle as the reference loops over an array (about
two minutes on eight cores):
  * per set and ReLU layer the number of inactive neurons, the number of crossing neurons and a 64-bit hash
    (blake2b of the little-endian int32 indices) of the crossing list in new-predicate order;
  * per set the estimated ranges of the output set;
  * per set and ReLU layer the classification margin min(|lb|, |ub|) over the layer's neurons, relative to the
    largest bound of the layer, and the neuron and bound at which it is reached; and every pre-ReLU bound whose
    magnitude is below 1e-6 of that scale (set, layer, neuron, lower / upper, value): the entries whose sign
    decides a classification.

Run from the repository root:  python tests/golden/make_fullsize_fixtures.py [4] [5]
"""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from nnv_amd.configs import make_config  # noqa: E402  (synthetic inputs and weights, no device needed)
from oracle import nnv_oracle as o  # noqa: E402

SAMPLES = 512
METHOD = "relax-star-area"


def flat(V):
    return V.reshape(-1, V.shape[-1], order="F") if V.ndim == 4 else V


def crossing_hash(idx):
    """64-bit hash of a crossing list in new-predicate order (what the test computes from the device's list)."""
    import hashlib
    return np.frombuffer(hashlib.blake2b(np.ascontiguousarray(idx, dtype="<i4").tobytes(), digest_size=8).digest(), dtype="<u8")[0]


NEAR_ZERO = 1e-6


def _cfg5_one(args):
    """One sub-box through the oracle: per ReLU layer (inactive, crossing, hash, margin, its neuron, its bound, scale,
    the near-zero bounds) and the output ranges."""
    i, lb, ub = args
    layers = _cfg5_one.layers
    S = o.star_from_box(lb, ub)
    per_layer = []
    for L in layers:
        if L["type"] == "relu":
            elb, eub = o.estimate_ranges(S)
            m1, m2 = o.relax_classify(elb, eub, METHOD)
            scale = max(np.max(np.abs(elb)), np.max(np.abs(eub)))
            both = np.concatenate([np.abs(elb), np.abs(eub)])
            k = int(np.argmin(both))
            vals = np.concatenate([elb, eub])
            near = np.flatnonzero(both < NEAR_ZERO * scale)
            per_layer.append((m1.size, m2.size, crossing_hash(m2), both[k] / scale, k % elb.size, k // elb.size, vals[k], scale,
                              [(int(j % elb.size), int(j // elb.size), float(vals[j])) for j in near]))
        S = o.nn_reach([L], S, METHOD, 1.0)
    olb, oub = o.output_ranges(S)
    return i, per_layer, np.asarray(olb).reshape(-1), np.asarray(oub).reshape(-1)


def _cfg5_init(layers):
    _cfg5_one.layers = layers
    try:
        from threadpoolctl import threadpool_limits
        _cfg5_one.limit = threadpool_limits(2)
    except Exception:
        pass


def main_cfg5(workers=4):
    import multiprocessing as mp
    cfg = make_config(5)
    boxes = o.box_partition(cfg["lb"], cfg["ub"], cfg["partition"]["indexes"], cfg["partition"]["numbers"])
    relu_layers = [li for li, L in enumerate(cfg["layers"]) if L["type"] == "relu"]
    n_sets, n_relu = len(boxes), len(relu_layers)
    inactive = np.zeros((n_sets, n_relu), dtype=np.int32)
    crossing = np.zeros((n_sets, n_relu), dtype=np.int32)
    hashes = np.zeros((n_sets, n_relu), dtype=np.uint64)
    margin = np.zeros((n_sets, n_relu))
    margin_neuron = np.zeros((n_sets, n_relu), dtype=np.int32)
    margin_upper = np.zeros((n_sets, n_relu), dtype=np.int8)
    margin_value = np.zeros((n_sets, n_relu))
    scale = np.zeros((n_sets, n_relu))
    near = []
    out_lb = np.zeros((n_sets, cfg["layers"][-1]["W"].shape[0]))
    out_ub = np.zeros_like(out_lb)
    t0 = time.time()
    with mp.Pool(workers, initializer=_cfg5_init, initargs=(cfg["layers"],)) as pool:
        for done, (i, per_layer, olb, oub) in enumerate(pool.imap_unordered(_cfg5_one, [(i, b[0], b[1]) for i, b in enumerate(boxes)],
                                                                             chunksize=4)):
            for r, (ni, m, h, mg, neuron, upper, val, sc, nz) in enumerate(per_layer):
                inactive[i, r], crossing[i, r], hashes[i, r] = ni, m, h
                margin[i, r], margin_neuron[i, r], margin_upper[i, r], margin_value[i, r], scale[i, r] = mg, neuron, upper, val, sc
                near.extend((i, r, nn_, up, v) for (nn_, up, v) in nz)
            out_lb[i], out_ub[i] = olb, oub
            if (done + 1) % 64 == 0:
                print("  %d / %d sets, %.0f s" % (done + 1, n_sets, time.time() - t0), flush=True)
    near.sort()
    data = {"relu_layers": np.array(relu_layers, dtype=np.int64), "inactive": inactive, "crossing": crossing, "crossing_hash": hashes,
            "margin": margin, "margin_neuron": margin_neuron, "margin_upper": margin_upper, "margin_value": margin_value,
            "scale": scale, "out_lb": out_lb, "out_ub": out_ub,
            "near_zero_where": np.array([(a, b, c, d) for (a, b, c, d, _) in near], dtype=np.int32).reshape(-1, 4),
            "near_zero_value": np.array([v for (_, _, _, _, v) in near], dtype=np.float64)}
    path = os.path.join(ROOT, "tests", "golden", "cfg5_fullsize_relax_star_area.npz")
    np.savez_compressed(path, **data)
    print("wrote", path, os.path.getsize(path), "bytes; smallest margin per ReLU layer:", margin.min(axis=0), "near-zero bounds:", len(near))


def main():
    cfg = make_config(4)
    sh = cfg["image_shape"]
    lb = cfg["lb"].reshape(sh, order="F")
    ub = cfg["ub"].reshape(sh, order="F")
    inp = o.image_star_from_bounds(lb, ub)
    t0 = time.time()
    out, sets = o.nn_reach(cfg["layers"], inp, METHOD, 1.0, keep=True)
    print("oracle reach: %.1f s" % (time.time() - t0))
    data = {"n_layers": np.array([len(cfg["layers"])], dtype=np.int64)}
    prev = inp
    for li, (L, s) in enumerate(zip(cfg["layers"], sets)):
        V = flat(s.V)
        rs = np.random.RandomState(4000 + li)
        rows = rs.randint(0, V.shape[0], size=SAMPLES)
        cols = rs.randint(0, V.shape[1], size=SAMPLES)
        cols[:32] = 0  # the centre column is always among the samples
        data["shape_%d" % li] = np.array(V.shape, dtype=np.int64)
        data["rows_%d" % li] = rows.astype(np.int64)
        data["cols_%d" % li] = cols.astype(np.int64)
        data["vals_%d" % li] = V[rows, cols].astype(np.float64)
        if L["type"] == "relu":
            pstar = prev.to_star() if isinstance(prev, o.OImageStar) else prev
            elb, eub = o.estimate_ranges(pstar)
            m1, m2 = o.relax_classify(elb, eub, METHOD)
            data["inactive_%d" % li] = np.array([m1.size], dtype=np.int64)
            data["crossing_%d" % li] = np.asarray(m2, dtype=np.int32)
        prev = s
    olb, oub = o.output_ranges(out)
    data["out_lb"] = np.asarray(olb, dtype=np.float64).reshape(-1)
    data["out_ub"] = np.asarray(oub, dtype=np.float64).reshape(-1)
    path = os.path.join(ROOT, "tests", "golden", "cfg4_fullsize_relax_star_area.npz")
    np.savez_compressed(path, **data)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    which = sys.argv[1:] or ["4", "5"]
    if "4" in which:
        main()
    if "5" in which:
        main_cfg5()

"""Write one benchmark configuration as a MATLAB v5 .mat file for nnv_amd/matlab/nnv_cpu_reach.m.

    python -m nnv_amd.export_fixture <k> <out.mat> [shrink]
"""
import sys

import numpy as np
import scipy.io as sio

from .configs import make_config


def main(argv):
    k = int(argv[1])
    out = argv[2]
    shrink = int(argv[3]) if len(argv) > 3 else 1
    cfg = make_config(k, shrink)
    layers = np.empty(len(cfg["layers"]), dtype=object)
    for i, L in enumerate(cfg["layers"]):
        d = {"type": L["type"]}
        for key in ("W", "b", "padding", "stride", "dilation"):
            if key in L:
                d[key] = np.asarray(L[key], dtype=np.float64)
        layers[i] = d
    data = {"layers": layers, "lb": cfg["lb"], "ub": cfg["ub"],
            "image_shape": np.asarray(cfg.get("image_shape", []), dtype=np.float64), "name": cfg["name"]}
    if "partition" in cfg:
        data["partition_indexes"] = np.asarray(cfg["partition"]["indexes"], dtype=np.float64) + 1  # 1-based
        data["partition_numbers"] = np.asarray(cfg["partition"]["numbers"], dtype=np.float64)
    sio.savemat(out, data, do_compression=True)
    print("wrote", out)


if __name__ == "__main__":
    main(sys.argv)

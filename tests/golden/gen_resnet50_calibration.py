"""Generates tests/golden/resnet50_calibration.json: the activation range
[min, max] at every observer point of the random-init ResNet-50 workload
(workloads.py), from one float forward over a seeded calibration batch.

Run here (CPU, needs torch only as a float conv routine):
    python tests/golden/gen_resnet50_calibration.py
The float forward is a calibration aid, not a parity reference: any float
convolution gives the same ranges to within rounding.
"""

import json
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

# workloads.py imports the hip package; only its pure-numpy helpers are used here
import workloads as W  # noqa: E402


def main():
    torch.manual_seed(0)
    params = W.resnet50_float_params(seed=0)
    rng = np.random.default_rng(5)
    x = torch.from_numpy(rng.uniform(0, 1, (8, 3, 224, 224)).astype(np.float32))
    ranges = {"input": [float(x.min()), float(x.max())]}
    specs = {c[0]: c for c in W.resnet50_convs()}

    def conv(name, t):
        _n, _ci, _co, _k, s, p, relu = specs[name]
        w, b = params[name]
        y = F.conv2d(t, torch.from_numpy(w), torch.from_numpy(b), s, p)
        if relu:
            y = F.relu(y)
        ranges[name] = [float(y.min()), float(y.max())]
        return y

    t = conv("conv1", x)
    t = F.max_pool2d(t, 3, 2, 1)
    for si, (_planes, blocks, _stride) in enumerate(W.STAGES, start=1):
        for b in range(blocks):
            p = f"layer{si}.{b}"
            idt = conv(f"{p}.downsample", t) if b == 0 else t
            o = conv(f"{p}.conv3", conv(f"{p}.conv2", conv(f"{p}.conv1", t)))
            t = F.relu(o + idt)
            ranges[f"{p}.add"] = [float(t.min()), float(t.max())]
    t = F.adaptive_avg_pool2d(t, 1).flatten(1)
    wfc, bfc = params["fc"]
    y = t @ torch.from_numpy(wfc).T + torch.from_numpy(bfc)
    ranges["fc"] = [float(y.min()), float(y.max())]
    out = {"about": "float activation ranges of the random-init ResNet-50 workload "
                    "(seed 0), calibration batch 8 x 3 x 224 x 224 uniform[0,1] seed 5",
           "ranges": ranges}
    path = os.path.join(ROOT, "tests", "golden", "resnet50_calibration.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path, len(ranges), "observer points")


if __name__ == "__main__":
    main()

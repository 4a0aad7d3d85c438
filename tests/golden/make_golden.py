"""Writes tests/golden/*.json.  The reference holds no golden vectors for this
path (its only check is run-time equality with NCCL), so these come from the
closed forms stated in oracle/ll128.py and oracle/ring.py, hand-checkable at
these sizes.  Run from the repository root: python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ll128, ring  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def ll128_cases():
    cases = []
    for layout, n, base, stride in ((0, 240, 7, 1), (0, 250, 1, 1), (0, 16, 1, 0),
                                    (1, 960, 100, 1), (1, 1000, 1, 1), (1, 8, 3, 0)):
        raw = ((np.arange(n) * 37 + 11) % 256).astype(np.uint8)
        msg = ll128.pack(raw, base, layout, stride)
        cases.append({"layout": layout, "flag_base": base, "flag_stride": stride,
                      "raw": raw.tolist(), "msg": msg.tolist()})
    return {"cases": cases}


def fold_cases():
    # fp16 values where the ring order is visible in the result
    cases = []
    rows = [[2048.0, 1.0, 1.0, 0.5], [1.0, 2048.0, 0.5, 1.0], [1.0, 1.0, 2048.0, 1.0],
            [0.5, 1.0, 1.0, 2048.0]]
    xs = [np.array(r, dtype=np.float16) for r in rows]
    for root in range(4):
        out = ring.reduce([x.view(np.uint8) for x in xs], root, "f16")[root]
        cases.append({"root": root, "rows_f16_bits": [x.view(np.uint16).tolist() for x in xs],
                      "result_f16_bits": out.view(np.uint16).tolist()})
    return {"cases": cases}


if __name__ == "__main__":
    with open(os.path.join(HERE, "ll128_vectors.json"), "w") as f:
        json.dump(ll128_cases(), f)
    with open(os.path.join(HERE, "fold_vectors.json"), "w") as f:
        json.dump(fold_cases(), f, indent=1)
    print("written")

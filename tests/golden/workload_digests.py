"""Writes tests/golden/workload_digests.json: valid-token counts, first sequence
lengths and sha256 digests of the seeded synthetic workloads, so that a change in the
generator (draw order, dtype casts) is caught.  Run from the repo root:
    python tests/golden/workload_digests.py
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import et_oracle as o  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    out = {}
    for name, wl in o.WORKLOADS.items():
        w = o.make_workload(name, layers=1)
        out[name] = dict(
            T=int(w["mask"].sum()), total=int(w["mask"].size),
            lens_first8=[int(v) for v in w["lens"][:8]],
            mask_sha256=sha(w["mask"]),
            x_first_row_sha256=sha(w["x"][0, 0]),
            layer0_wq_row0_sha256=sha(w["weights"][0][0]),
            layer0_out_kernel_row0_sha256=sha(w["weights"][12][0]),
        )
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "workload_digests.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print(json.dumps({k: v["T"] for k, v in out.items()}))


if __name__ == "__main__":
    main()

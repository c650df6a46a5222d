"""Writes tests/golden/config2.json and config2_masks.npy (pattern-discovery configuration 2).

Runs the oracle only (no reference code).  For seeds 0, 1, 2, ... it builds the two 1024x1024 score maps,
computes the masks along the float32 PyTorch route and the float64 closed-form route, measures the
relative difference of the two pooled maps and the decision margin of every comparison the walks make,
and keeps the first seed for which the margin exceeds 8x the route difference and the masks agree.
Rejected seeds are listed in the JSON.

    python tests/golden/make_config2.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import pattern as op  # noqa: E402
from spion_amd import workloads  # noqa: E402

Q, BS, L = 0.90, 32, 1024


def main():
    rejected = []
    for seed in range(64):
        maps = workloads.score_maps_config2(2, L, 32, seed=seed).numpy()
        ok, masks, margins, errs = True, [], [], []
        for i in range(2):
            m64, p64, t64 = op.generate_mask_conv_ff(maps[i], BS, Q, route="fp64")
            m32, p32, t32 = op.generate_mask_conv_ff(maps[i], BS, Q, route="torch")
            err = float(np.max(np.abs(p64.astype(np.float64) - p32) / np.abs(p64)))
            margin = op.decision_margin(p64, Q)
            margins.append(margin)
            errs.append(err)
            masks.append(m64)
            ok = ok and margin > 8 * err and np.array_equal(m64, m32)
        print(f"seed {seed}: margins {margins} route errors {errs} -> {'ok' if ok else 'rejected'}", flush=True)
        if ok:
            np.save(os.path.join(HERE, "config2_masks.npy"), np.stack(masks).astype(np.int8))
            meta = dict(seed=seed, quantile=Q, block_size=BS, seq_len=L, decision_margin=margins,
                        fp32_route_rel_error=errs, rejected_seeds=rejected,
                        blocks_set=[int(m.sum()) for m in masks])
            json.dump(meta, open(os.path.join(HERE, "config2.json"), "w"), indent=1)
            return
        rejected.append(dict(seed=seed, decision_margin=margins, fp32_route_rel_error=errs))
    raise SystemExit("no seed passed the margin screen")


if __name__ == "__main__":
    main()

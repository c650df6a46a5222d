"""Writes tests/golden/config2.json and config2_masks.npy (pattern-discovery configuration 2).

Runs the oracle only (no reference code).  For every seed of a range it builds the two 1024x1024 score maps and
measures the decision margin: the smallest relative gap over every comparison the path walks make (down > right,
. > diagonal, . > threshold) on the float64-route pooled map.  It keeps the seed with the largest margin, then
checks on that seed that the float32 PyTorch route (the reference's: F.conv2d, avg_pool2d, torch.quantile) and
the float64 closed-form route give the same masks and that the margin exceeds 100 times the relative difference
between the two routes' pooled maps -- so any correct summation order yields the identical mask.

A walk makes about ten thousand comparisons per map, so margins above 1e-3 are out of reach: over seeds 0..2999
the best is 6.3e-4 (seed 2608), the median 2e-5.  The float32 route differs from the float64 one by about 2e-6.

The three runners-up of the scan (the next largest margins) get the same treatment: their masks go to
config2_more_masks.npy ([3, 2, 32, 32]) and their seeds, margins and route errors to "more" in config2.json.

    python tests/golden/make_config2.py [first_seed last_seed]      (default 0 3000: about a quarter of an hour on 8 cores)
    python tests/golden/make_config2.py more                        (only the runners-up of the scan already on file)
"""
import json
import os
import sys
from multiprocessing import Pool

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import pattern as op  # noqa: E402
from spion_amd import workloads  # noqa: E402

Q, BS, L = 0.90, 32, 1024
MIN_FACTOR = 100.0


def margins_of(seed):
    maps = workloads.score_maps_config2(2, L, 32, seed=seed).numpy()
    return seed, [op.decision_margin(op.pooled_map(maps[i], BS, 31, "fp64"), Q) for i in range(2)]


def masks_of(seed, margins):
    """Masks of one seed's two maps, after checking that both routes agree and the margin dwarfs their difference."""
    maps = workloads.score_maps_config2(2, L, 32, seed=seed).numpy()
    masks, errs = [], []
    for i in range(2):
        m64, p64, _ = op.generate_mask_conv_ff(maps[i], BS, Q, route="fp64")
        m32, p32, _ = op.generate_mask_conv_ff(maps[i], BS, Q, route="torch")
        errs.append(float(np.max(np.abs(p64.astype(np.float64) - p32) / np.abs(p64))))
        if not np.array_equal(m64, m32):
            raise SystemExit(f"seed {seed}: the float32 and float64 routes disagree on map {i}")
        masks.append(m64)
    if min(margins) <= MIN_FACTOR * max(errs):
        raise SystemExit(f"seed {seed}: margin {min(margins):.3e} is not {MIN_FACTOR:g}x the route error {max(errs):.3e}")
    return masks, errs


def write_more():
    path = os.path.join(HERE, "config2.json")
    meta = json.load(open(path))
    more, stack = [], []
    for r in meta["runners_up"][:3]:
        masks, errs = masks_of(r["seed"], r["decision_margin"])
        stack.append(np.stack(masks))
        more.append(dict(seed=r["seed"], decision_margin=r["decision_margin"], fp32_route_rel_error=errs,
                         blocks_set=[int(m.sum()) for m in masks]))
    np.save(os.path.join(HERE, "config2_more_masks.npy"), np.stack(stack).astype(np.int8))
    meta["more"] = more
    json.dump(meta, open(path, "w"), indent=1)
    print(json.dumps(more, indent=1))


def main():
    if sys.argv[1:] == ["more"]:
        write_more()
        return
    lo, hi = (int(sys.argv[1]), int(sys.argv[2])) if len(sys.argv) == 3 else (0, 3000)
    with Pool(min(8, os.cpu_count() or 1)) as pool:
        scan = pool.map(margins_of, range(lo, hi), chunksize=8)
    scan.sort(key=lambda r: -min(r[1]))
    seed, margins = scan[0]
    masks, errs = masks_of(seed, margins)
    np.save(os.path.join(HERE, "config2_masks.npy"), np.stack(masks).astype(np.int8))
    all_min = sorted(min(r[1]) for r in scan)
    meta = dict(seed=seed, quantile=Q, block_size=BS, seq_len=L, decision_margin=margins,
                fp32_route_rel_error=errs, margin_over_route_error=min(margins) / max(errs),
                seeds_scanned=[lo, hi], median_margin_of_scan=all_min[len(all_min) // 2],
                runners_up=[dict(seed=s, decision_margin=m) for s, m in scan[1:6]],
                blocks_set=[int(m.sum()) for m in masks])
    json.dump(meta, open(os.path.join(HERE, "config2.json"), "w"), indent=1)
    print(json.dumps(meta, indent=1))
    write_more()


if __name__ == "__main__":
    main()

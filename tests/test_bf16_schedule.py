"""The schedule of the bf16 kernels (host logic of libspion_hip.so, spion_debug_bf16_plan: no device needed).

A launch is a fixed set of persistent wavefronts; each walks a list of {head, item}.  Whatever the pattern, every tile
of every strip of every head must be walked exactly once, chunks of a long strip must cover it without gaps and own
distinct workspace slots, pairs must only join strips with the same number of tiles, a die's lanes must only see the
heads of that die, and no lane may carry much more than its share."""
import ctypes
import zlib

import numpy as np
import pytest

from spion_amd import _lib


def _plan(ptr, pairs, NB, lanes):
    core = _lib.core()
    core.spion_debug_bf16_plan.restype = ctypes.c_int
    ptr = np.ascontiguousarray(ptr, dtype=np.int32)
    nstrips = ptr.size - 1
    counts = (ctypes.c_int * 4)()
    P = ctypes.POINTER(ctypes.c_int)
    as_p = lambda a: a.ctypes.data_as(P)
    n_lanes = core.spion_debug_bf16_plan(as_p(ptr), nstrips, int(pairs), NB, lanes, None, 0, None, 0, None, 0, None, 0, counts)
    assert n_lanes > 0
    items = np.zeros(max(counts[0], 1), np.int32)
    lane_ptr = np.zeros(n_lanes + 1, np.int32)
    lane_ent = np.zeros(max(counts[1], 1), np.int32)
    longs = np.zeros(max(counts[2], 1), np.int32)
    again = core.spion_debug_bf16_plan(as_p(ptr), nstrips, int(pairs), NB, lanes, as_p(items), items.size, as_p(lane_ptr),
                                       lane_ptr.size, as_p(lane_ent), lane_ent.size, as_p(longs), longs.size, counts)
    assert again == n_lanes
    return dict(lanes=n_lanes, items=items[: counts[0]].reshape(-1, 4), lane_ptr=lane_ptr,
                ents=lane_ent[: counts[1]].reshape(-1, 2), longs=longs[: counts[2]].reshape(-1, 4), slots=counts[3])


def _tile_ptr(rng, nstrips, kind, pairs):
    if kind == "band":
        cnt = np.minimum(np.arange(nstrips) + 3, 5) + rng.integers(0, 4, nstrips)
    elif kind == "global":
        cnt = rng.integers(2, 9, nstrips)
        cnt[rng.integers(nstrips)] = nstrips          # a strip that holds every tile column
    elif kind == "empty":
        cnt = rng.integers(0, 3, nstrips)
    else:
        cnt = rng.integers(1, 40, nstrips)
    if pairs:                                          # strips 2p and 2p+1 hold the same tiles
        cnt = np.repeat(cnt[::2], 2)[:nstrips]
    return np.concatenate([[0], np.cumsum(cnt)]).astype(np.int32)


@pytest.mark.parametrize("kind", ["band", "global", "empty", "random"])
@pytest.mark.parametrize("pairs", [False, True])
@pytest.mark.parametrize("NB,lanes", [(32, 2048), (5, 2048), (8, 24), (3, 3), (16, 1)])
def test_schedule_walks_every_tile_once(kind, pairs, NB, lanes):
    rng = np.random.default_rng(zlib.crc32(repr((kind, pairs, NB, lanes)).encode()))
    nstrips = int(rng.choice([2, 8, 64, 512]))
    ptr = _tile_ptr(rng, nstrips, kind, pairs)
    plan = _plan(ptr, pairs, NB, lanes)
    items, ents, lane_ptr = plan["items"], plan["ents"], plan["lane_ptr"]
    groups = 8 if NB % 8 == 0 else 1
    assert plan["lanes"] % groups == 0 and plan["lanes"] >= groups
    assert lane_ptr[0] == 0 and lane_ptr[-1] == len(ents) and np.all(np.diff(lane_ptr) >= 0)
    # every (head, item) once
    seen = np.zeros((NB, len(items)), np.int32)
    np.add.at(seen, (ents[:, 0], ents[:, 1]), 1)
    assert np.all(seen == 1)
    # the items cover every strip's tiles exactly once
    cover = np.zeros(int(ptr[-1]) + 1, np.int32)
    slots = []
    for strip, t0, n, kind_ in items:
        assert n >= 0 and ptr[strip] <= t0 and t0 + n <= ptr[strip + 1]
        if kind_ == -2:
            assert pairs and strip % 2 == 0 and ptr[strip + 2] - ptr[strip + 1] == n == ptr[strip + 1] - ptr[strip]
            cover[ptr[strip]: ptr[strip + 2]] += 1
        else:
            cover[t0: t0 + n] += 1
            if kind_ >= 0:
                slots.append(int(kind_))
            else:
                assert kind_ == -1 and n == ptr[strip + 1] - ptr[strip]
    assert np.all(cover[: int(ptr[-1])] == 1)
    assert sorted(slots) == list(range(plan["slots"]))
    # long strips: consecutive slots, chunks in tile order
    for strip, first, chunks, tiles in plan["longs"]:
        mine = [(t0, n) for s_, t0, n, k_ in items if s_ == strip and first <= k_ < first + chunks]
        assert len(mine) == chunks and sum(n for _, n in mine) == tiles == ptr[strip + 1] - ptr[strip]
    # a die's lanes see only that die's heads, one head after the other
    per_die = NB // groups
    for lane in range(plan["lanes"]):
        heads = ents[lane_ptr[lane]: lane_ptr[lane + 1], 0]
        assert np.all(heads // per_die == lane % groups) if groups == 8 else True
        assert np.all(np.diff(heads) >= 0)
    # balance: no lane carries more than its die's average plus one longest item
    w = np.where(items[:, 3] == -2, 2, 1) * items[:, 2] + 2
    load = np.array([w[ents[lane_ptr[l]: lane_ptr[l + 1], 1]].sum() for l in range(plan["lanes"])])
    for g in range(groups):
        mine = load[g::groups]
        assert mine.max() <= mine.mean() + w.max() + 1e-9


def test_schedule_rejects_bad_arguments():
    core = _lib.core()
    core.spion_debug_bf16_plan.restype = ctypes.c_int
    ptr = (ctypes.c_int * 3)(0, 1, 2)
    assert core.spion_debug_bf16_plan(None, 2, 0, 4, 8, None, 0, None, 0, None, 0, None, 0, None) == -1
    assert core.spion_debug_bf16_plan(ptr, 2, 0, 0, 8, None, 0, None, 0, None, 0, None, 0, None) == -1
    assert core.spion_debug_bf16_plan(ptr, 2, 0, 4, 0, None, 0, None, 0, None, 0, None, 0, None) == -1

"""Writes tests/golden/routing_fixtures.npz: small input/output vectors for the integer stages.

Expected outputs come from numpy library routines only (bincount, cumsum, stable argsort) -- neither the oracle nor the
HIP library nor the reference is involved, so the fixtures pin both sides independently.

    python tests/golden/make_fixtures.py
"""

import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def main() -> None:
    out = {}
    # C1 of the baseline: 65,536 ids uniform in [0, 64) from seed 42 -- only the 64 counts / offsets are stored
    rng = np.random.default_rng(42)
    ids = rng.integers(0, 64, size=65536, dtype=np.int64)
    counts = np.bincount(ids, minlength=64).astype(np.uint32)
    out["c1_seed"] = np.array([42])
    out["c1_counts"] = counts
    out["c1_ends"] = np.cumsum(counts).astype(np.uint32)
    out["c1_starts"] = (np.cumsum(counts) - counts).astype(np.uint32)
    # a small ragged case with empty experts, stored in full
    rng = np.random.default_rng(7)
    ids = rng.choice(np.array([0, 2, 3, 7, 11]), size=300).astype(np.int64)
    out["small_ids"] = ids
    out["small_num_experts"] = np.array([13])
    out["small_counts"] = np.bincount(ids, minlength=13).astype(np.uint32)
    order = np.argsort(ids, kind="stable")
    out["small_sorted_scattered_idxs"] = order.astype(np.int32)
    out["small_sorted_expert_idxs"] = ids[order].astype(np.int32)
    np.savez(os.path.join(HERE, "routing_fixtures.npz"), **out)


if __name__ == "__main__":
    main()

"""The invariants the reference's test checks on the outputs of moe_create_indices
(max/kernels/test/gpu/nn/test_moe_indices.mojo:38-140), restated with numpy."""
import numpy as np


def check_indices(topk_ids, num_experts, order, start, restore, expert_ids, stats):
    ids = np.asarray(topk_ids, dtype=np.int64)
    n = ids.shape[0]
    counts = np.bincount(ids, minlength=num_experts) if n else np.zeros(num_experts, dtype=np.int64)
    order, start, restore = order.astype(np.int64), start.astype(np.int64), restore.astype(np.int64)
    # every assignment appears once, and assignments of one expert are contiguous
    assert np.array_equal(np.sort(order), np.arange(n))
    grouped = ids[order]
    changes = np.flatnonzero(np.diff(grouped)) + 1
    runs = np.split(grouped, changes) if n else []
    assert len({int(r[0]) for r in runs}) == len(runs), "tokens are grouped incorrectly"
    # stats: most frequent expert; one slot per expert
    assert int(stats[0]) == (int(counts.max()) if n else 0)
    assert int(stats[1]) == num_experts
    # start indices against expert_ids
    assert start[0] == 0 and start[-1] == n and np.all(np.diff(start) >= 0)
    assert sorted(expert_ids.tolist()) == list(range(num_experts))
    for z in range(int(stats[1])):
        seg = grouped[start[z]:start[z + 1]]
        assert np.all(seg == expert_ids[z]), "expert range in start indices is incorrect"
        assert len(seg) == counts[expert_ids[z]]
    # the restore permutation
    assert np.array_equal(order[restore], np.arange(n)), "restore token order is incorrect"

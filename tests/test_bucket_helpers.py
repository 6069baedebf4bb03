"""Host logic of the bucket loop, on the CPU: which edges are held out, which
are trained, and which single-relation batches a bucket is cut into."""
import torch


def test_train_edge_indices_is_the_reference_assignment(pbg):
    """train_cpu.py:852-856, restated literally (sequential index assignment, so a
    held-out edge that was drawn twice keeps its last slot), duplicates included."""
    bl = pbg.bucket_loop
    g = torch.Generator().manual_seed(0)
    for n, num_eval in ((10, 2), (10, 3), (1000, 300), (50, 50), (7, 1), (2000, 1900)):
        for _ in range(5):
            eval_idx = torch.randint(n, (num_eval,), generator=g)
            num_train = n - num_eval
            want = torch.arange(n)
            want[eval_idx] = torch.arange(num_train, n)
            want = want[:num_train]
            got = bl.train_edge_indices(n, eval_idx)
            assert torch.equal(got, want)
    # the cases worked out by hand
    assert bl.train_edge_indices(10, torch.tensor([2, 9])).tolist() == [0, 1, 8, 3, 4, 5, 6, 7]
    assert bl.train_edge_indices(10, torch.tensor([2, 2, 9])).tolist() == [0, 1, 8, 3, 4, 5, 6]
    assert bl.train_edge_indices(5, None).tolist() == [0, 1, 2, 3, 4]


def test_holdout_indices(pbg):
    bl = pbg.bucket_loop
    b = bl.Bucket(1, 2)
    assert bl.holdout_indices(1000, 0.0, b) is None
    assert bl.holdout_indices(10, 0.05, b) is None  # int(0.5) = 0 edges
    a = bl.holdout_indices(1000, 0.05, b)
    assert a.shape == (50,) and a.dtype == torch.int64 and int(a.min()) >= 0 and int(a.max()) < 1000
    assert torch.equal(a, bl.holdout_indices(1000, 0.05, b))  # the same edges every epoch
    assert not torch.equal(a, bl.holdout_indices(1000, 0.05, bl.Bucket(2, 1)))
    # the draw of train_cpu.py:664-671 for this bucket
    g = torch.Generator()
    g.manual_seed(hash((0, 0, 1, 2)))
    assert torch.equal(a, torch.randint(1000, (50,), dtype=torch.long, generator=g))


def test_plan_relation_batches(pbg):
    bl = pbg.bucket_loop
    sizes = [5, 0, 12, 1, 40]
    plan = bl.plan_relation_batches(sizes, 4, torch.Generator().manual_seed(1))
    seen = {g: 0 for g in range(len(sizes))}
    for group, offset, length in plan:  # every group is consumed front to back, in full batches until its end
        assert offset == seen[group]
        assert length == min(4, sizes[group] - offset) and length > 0
        seen[group] += length
    assert [seen[g] for g in range(len(sizes))] == sizes
    # the first batch comes from a group with probability proportional to its size
    first = [bl.plan_relation_batches([30, 10], 50, torch.Generator().manual_seed(s))[0][0] for s in range(400)]
    assert 0.65 < first.count(0) / 400 < 0.85
    assert bl.plan_relation_batches([], 4) == [] and bl.plan_relation_batches([0, 0], 4) == []

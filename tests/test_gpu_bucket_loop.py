"""Partition swap and the per-bucket loop: the result does not depend on how
many partitions stay resident in HBM, and it matches the CPU oracle run over
the same buckets, edge order and negatives."""
import random

import pytest
import torch

from oracle import step as ostep

DEV = "cuda:0"


def make_graph(nparts, rows, dim, edges_per_bucket, seed):
    g = torch.Generator().manual_seed(seed)
    tables = {p: torch.randn(rows + 3 * p, dim, generator=g) * 0.1 for p in range(nparts)}
    edges = {}
    for lhs in range(nparts):
        for rhs in range(nparts):
            n = edges_per_bucket + 17 * lhs + 5 * rhs
            edges[(lhs, rhs)] = (torch.randint(0, rows + 3 * lhs, (n,), generator=g),
                                 torch.randint(0, rows + 3 * rhs, (n,), generator=g),
                                 torch.zeros(n, dtype=torch.int64))
    return tables, edges


def run_loop(pbg, tables, edges, nparts, dim, resident, hooks=None, **kw):
    bl = pbg.bucket_loop
    store = bl.PartitionStore()
    for p, t in tables.items():
        store.add(("e", p), t)
    loop = bl.BucketLoop(store, {bl.Bucket(l, r): e for (l, r), e in edges.items()}, lhs_entity="e", rhs_entity="e",
                         nparts_lhs=nparts, nparts_rhs=nparts, dim=dim, resident_partitions=resident, seed=3,
                         **(hooks or {}), **kw)
    stats = [loop.train_epoch() for _ in range(2)]
    return store, stats, loop


@pytest.mark.gpu
def test_result_independent_of_residency(pbg):
    nparts, dim = 3, 16
    tables, edges = make_graph(nparts, 400, dim, 700, seed=1)
    kw = dict(batch_size=100, num_workers=3, num_batch_negs=10, num_uniform_negs=10, loss="softmax")
    a, sa, la = run_loop(pbg, tables, edges, nparts, dim, 2, **kw)
    b, sb, lb = run_loop(pbg, tables, edges, nparts, dim, 3, **kw)
    c, sc, lc = run_loop(pbg, tables, edges, nparts, dim, 6, **kw)
    for p in range(nparts):
        assert not torch.equal(a.tables[("e", p)], tables[p])
        for other in (b, c):
            assert torch.equal(a.tables[("e", p)], other.tables[("e", p)])
            assert torch.equal(a.sums[("e", p)], other.sums[("e", p)])
    assert [s.loss for e in sa for s in e] == [s.loss for e in sc for s in e]
    # two buffers reload partitions, six never write back before the flush
    assert la.cache.bytes_uploaded > lc.cache.bytes_uploaded


@pytest.mark.gpu
def test_bucket_loop_matches_oracle(pbg):
    nparts, dim, bsz, workers, nb, nu = 2, 12, 50, 2, 10, 5
    tables, edges = make_graph(nparts, 300, dim, 260, seed=2)
    drawn = []

    def negatives(k, c, u, rows, generator, device):
        t = torch.randint(0, rows, (k, c, u), generator=generator, device=device)
        drawn.append(t.cpu())
        return t

    perms = {}

    def edge_order(bucket, n):
        perms.setdefault((bucket.lhs, bucket.rhs), []).append(torch.randperm(n, generator=torch.Generator().manual_seed(n)))
        return perms[(bucket.lhs, bucket.rhs)][-1]

    store, stats, loop = run_loop(pbg, tables, edges, nparts, dim, 2, hooks=dict(negatives=negatives, edge_order=edge_order),
                                  batch_size=bsz, num_workers=workers, num_batch_negs=nb, num_uniform_negs=nu,
                                  loss="softmax", bucket_order="lexicographic")
    cfg = ostep.StepConfig(dim=dim, loss="softmax", num_batch_negs=nb, num_uniform_negs=nu, lr=0.1)
    w = {p: t.clone() for p, t in tables.items()}
    g = {p: torch.zeros(t.shape[0]) for p, t in tables.items()}
    it = iter(drawn)
    want_loss = []
    for epoch in range(2):
        for lhs_p in range(nparts):
            for rhs_p in range(nparts):
                lhs, rhs, _ = edges[(lhs_p, rhs_p)]
                perm = perms[(lhs_p, rhs_p)][epoch]
                lhs, rhs = lhs[perm], rhs[perm]
                st = ostep.make_state(cfg, w[lhs_p], None if lhs_p == rhs_p else w[rhs_p])
                st.g_lhs = g[lhs_p]
                st.g_rhs = g[lhs_p] if lhs_p == rhs_p else g[rhs_p]
                n, off, total = lhs.shape[0], 0, 0.0
                while off < n:
                    left = n - off
                    k, b_now = (min(workers, left // bsz), bsz) if left >= bsz else (1, left)
                    ul, ur = next(it), next(it)
                    batches = [(lhs[off + i * b_now: off + (i + 1) * b_now], rhs[off + i * b_now: off + (i + 1) * b_now],
                                0, ul[i], ur[i]) for i in range(k)]
                    total += sum(o.loss for o in ostep.train_lockstep(cfg, st, batches))
                    off += k * b_now
                want_loss.append(total)
    got_loss = [s.loss for e in stats for s in e]
    assert got_loss == pytest.approx(want_loss, rel=1e-4)
    for p in range(nparts):
        assert torch.allclose(store.tables[("e", p)], w[p], rtol=1e-4, atol=1e-6)
        assert torch.allclose(store.sums[("e", p)], g[p], rtol=1e-4, atol=1e-9)


def test_bucket_orders(pbg):
    bl = pbg.bucket_loop
    lex = bl.create_buckets_ordered_lexicographically(2, 3)
    assert [(b.lhs, b.rhs) for b in lex] == [(0, 0), (0, 1), (0, 2), (1, 0), (1, 1), (1, 2)]
    for order in ("inside_out", "outside_in", "random", "lexicographic"):
        got = bl.create_ordered_buckets(3, 4, order, generator=random.Random(0))
        assert sorted((b.lhs, b.rhs) for b in got) == [(l, r) for l in range(3) for r in range(4)]
    out_in = bl.create_ordered_buckets(3, 4, "outside_in", generator=random.Random(0))
    layers = [min(b.lhs, b.rhs) for b in out_in]
    assert layers == sorted(layers) and layers.count(0) == 6 and layers.count(1) == 4 and layers.count(2) == 2
    in_out = bl.create_ordered_buckets(3, 4, "inside_out", generator=random.Random(0))
    assert [min(b.lhs, b.rhs) for b in in_out] == sorted(layers, reverse=True)
    with pytest.raises(NotImplementedError):
        bl.create_ordered_buckets(2, 2, "affinity", generator=random.Random(0))

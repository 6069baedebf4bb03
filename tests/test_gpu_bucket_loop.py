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


def _calls_of(n, bsz, workers):
    """(offset, batches, batch length) of the calls that cut n consecutive edges."""
    out, off = [], 0
    while off < n:
        left = n - off
        k, b_now = (min(workers, left // bsz), bsz) if left >= bsz else (1, left)
        out.append((off, k, b_now))
        off += k * b_now
    return out


def _oracle_eval(cfg_eval, st, lhs, rhs, eval_idx, bsz, workers, draws):
    """RankingEvaluator's sums (eval.py:57-81) over the held-out edges on the
    oracle's scores, as (low, high) bounds: a negative that is the positive's own
    entity scores the same as the positive up to rounding, and which way such a tie
    falls differs between two fp32 implementations."""
    lhs, rhs = lhs[eval_idx], rhs[eval_idx]
    keys = ("pos_rank", "mrr", "r1", "r10")
    lo, hi = dict.fromkeys(keys, 0.0), dict.fromkeys(keys, 0.0)
    loss, count = 0.0, 0
    for off, k, b_now in _calls_of(lhs.shape[0], bsz, workers):
        ul, ur = next(draws), next(draws)
        for i in range(k):
            sl = slice(off + i * b_now, off + (i + 1) * b_now)
            out, _ = ostep.forward_backward(cfg_eval, st, lhs[sl], rhs[sl], 0, ul[i], ur[i], keep_scores=True)
            sc = out.scores
            loss += out.loss
            count += b_now
            for bound, sign in ((lo, -1.0), (hi, 1.0)):
                # low ranks: a near-tie does not count against the positive; high ranks: it does
                ranks = []
                for pos, neg in ((sc.lhs_pos, sc.lhs_neg), (sc.rhs_pos, sc.rhs_neg)):
                    tol = 1e-5 * (1.0 + pos.abs().unsqueeze(1))
                    ranks.append((neg >= pos.unsqueeze(1) - sign * tol).sum(1) + 1)
                mean2 = lambda a, b: (float(a.sum()) + float(b.sum())) / 2
                bound["pos_rank"] += mean2(*ranks)
                bound["mrr"] += mean2(*(r.float().reciprocal() for r in ranks))
                bound["r1"] += mean2(*(r.le(1) for r in ranks))
                bound["r10"] += mean2(*(r.le(10) for r in ranks))
    # low ranks give the high mrr / hits, and the other way round
    low = dict(pos_rank=lo["pos_rank"], mrr=hi["mrr"], r1=hi["r1"], r10=hi["r10"])
    high = dict(pos_rank=hi["pos_rank"], mrr=lo["mrr"], r1=lo["r1"], r10=lo["r10"])
    return dict(loss=loss, count=count, low=low, high=high)


@pytest.mark.gpu
def test_holdout_evaluation_matches_oracle(pbg):
    """eval_fraction: the held-out edges (train_cpu.py:661-672) are not trained on
    (:852-856) and are ranked before and after each bucket (:675,690) with the
    evaluation-time negatives; tables, losses and ranking sums against the oracle
    driven through the same sequence."""
    bl = pbg.bucket_loop
    nparts, dim, bsz, workers, nb, nu, enb, enu, frac = 2, 12, 50, 2, 10, 5, 20, 7, 0.2
    tables, edges = make_graph(nparts, 300, dim, 330, seed=5)
    drawn, perms = [], {}

    def negatives(k, c, u, rows, generator, device):
        t = torch.randint(0, rows, (k, c, u), generator=generator, device=device)
        drawn.append(t.cpu())
        return t

    def edge_order(bucket, n):
        perms.setdefault((bucket.lhs, bucket.rhs), []).append(torch.randperm(n, generator=torch.Generator().manual_seed(n)))
        return perms[(bucket.lhs, bucket.rhs)][-1]

    store, stats, loop = run_loop(pbg, tables, edges, nparts, dim, 2, hooks=dict(negatives=negatives, edge_order=edge_order),
                                  batch_size=bsz, num_workers=workers, num_batch_negs=nb, num_uniform_negs=nu,
                                  loss="softmax", bucket_order="lexicographic", eval_fraction=frac,
                                  eval_num_batch_negs=enb, eval_num_uniform_negs=enu)
    cfg = ostep.StepConfig(dim=dim, loss="softmax", num_batch_negs=nb, num_uniform_negs=nu, lr=0.1)
    cfg_eval = ostep.StepConfig(dim=dim, loss="softmax", num_batch_negs=enb, num_uniform_negs=enu, lr=0.1)
    ebsz = 60  # batch_size rounded up to a multiple of eval_num_batch_negs (train_cpu.py:887-889)
    w = {p: t.clone() for p, t in tables.items()}
    g = {p: torch.zeros(t.shape[0]) for p, t in tables.items()}
    it = iter(drawn)
    flat = [s for e in stats for s in e]
    pos = 0
    for epoch in range(2):
        for lhs_p in range(nparts):
            for rhs_p in range(nparts):
                got = flat[pos]
                pos += 1
                lhs, rhs, _ = edges[(lhs_p, rhs_p)]
                n = lhs.shape[0]
                eval_idx = bl.holdout_indices(n, frac, bl.Bucket(lhs_p, rhs_p))
                assert eval_idx.shape[0] == int(n * frac)
                st = ostep.make_state(cfg, w[lhs_p], None if lhs_p == rhs_p else w[rhs_p])
                st.g_lhs = g[lhs_p]
                st.g_rhs = g[lhs_p] if lhs_p == rhs_p else g[rhs_p]
                want_before = _oracle_eval(cfg_eval, st, lhs, rhs, eval_idx, ebsz, workers, it)
                # the training edges, by the reference's own statements
                num_train = n - eval_idx.shape[0]
                train_idx = torch.arange(n)
                train_idx[eval_idx] = torch.arange(num_train, n)
                order = train_idx[:num_train][perms[(lhs_p, rhs_p)][epoch]]
                assert got.num_edges == num_train
                tl, tr = lhs[order], rhs[order]
                total = 0.0
                for off, k, b_now in _calls_of(num_train, bsz, workers):
                    ul, ur = next(it), next(it)
                    batches = [(tl[off + i * b_now: off + (i + 1) * b_now], tr[off + i * b_now: off + (i + 1) * b_now],
                                0, ul[i], ur[i]) for i in range(k)]
                    total += sum(o.loss for o in ostep.train_lockstep(cfg, st, batches))
                want_after = _oracle_eval(cfg_eval, st, lhs, rhs, eval_idx, ebsz, workers, it)
                assert got.loss == pytest.approx(total, rel=1e-4)
                for have, want in ((got.eval_before, want_before), (got.eval_after, want_after)):
                    m = have.metrics
                    assert have.count == want["count"] == eval_idx.shape[0]
                    assert m["loss"] == pytest.approx(want["loss"], rel=1e-4)
                    for key in ("pos_rank", "mrr", "r1", "r10"):
                        assert want["low"][key] - 1e-3 <= m[key] <= want["high"][key] + 1e-3, key
                    assert want["high"]["pos_rank"] - want["low"]["pos_rank"] <= 0.2 * have.count  # the bounds bind
                    assert 0.0 <= have.average().metrics["auc"] <= 1.0
    assert next(it, None) is None  # every draw was accounted for
    for p in range(nparts):
        assert torch.allclose(store.tables[("e", p)], w[p], rtol=1e-4, atol=1e-6)
        assert torch.allclose(store.sums[("e", p)], g[p], rtol=1e-4, atol=1e-9)


@pytest.mark.gpu
def test_standard_relations_train_in_single_relation_batches(pbg):
    """Several standard (non-dynamic) relation types: every batch holds one type
    (batching.py:60-79), every training edge is used once, and the calls the loop
    made, replayed on the oracle, give the same tables and operator parameters."""
    bl = pbg.bucket_loop
    nparts, dim, bsz, workers, nb, nu, nrel = 2, 8, 40, 3, 10, 5, 3
    tables, edges = make_graph(nparts, 250, dim, 420, seed=7)
    g0 = torch.Generator().manual_seed(11)
    edges = {k: (l, r, torch.randint(0, nrel, l.shape, generator=g0) ** 2 % nrel) for k, (l, r, _) in edges.items()}
    cfg = ostep.StepConfig(dim=dim, operator="translation", loss="ranking", margin=0.1, num_batch_negs=nb,
                           num_uniform_negs=nu, num_relations=nrel, relation_weights=[1.0] * nrel, lr=0.1,
                           regularization_coef=0.01, global_emb=True)
    st0 = ostep.make_state(cfg, tables[0])
    for k in st0.rhs_op:
        st0.rhs_op[k] = st0.rhs_op[k] + 0.1 * torch.randn(st0.rhs_op[k].shape, generator=g0)
    rhs_op = {k: v.clone().to(DEV) for k, v in st0.rhs_op.items()}
    rhs_sum = {k: torch.zeros_like(v) for k, v in rhs_op.items()}
    glob0 = 0.05 * torch.randn(dim, generator=g0)
    glob_dev, glob_sum_dev = glob0.clone().to(DEV), torch.zeros(dim, device=DEV)
    drawn = []

    def negatives(k, c, u, rows, generator, device):
        t = torch.randint(0, rows, (k, c, u), generator=generator, device=device)
        drawn.append(t.cpu())
        return t

    store, stats, loop = run_loop(pbg, tables, edges, nparts, dim, 2, hooks=dict(negatives=negatives, record_calls=True),
                                  batch_size=bsz, num_workers=workers, num_batch_negs=nb, num_uniform_negs=nu,
                                  operator="translation", num_relations=nrel, rhs_op=rhs_op, rhs_op_sum=rhs_sum,
                                  bucket_order="lexicographic", regularization_coef=0.01,
                                  global_embs={"e": (glob_dev, glob_sum_dev)})
    w = {p: t.clone() for p, t in tables.items()}
    g = {p: torch.zeros(t.shape[0]) for p, t in tables.items()}
    op = {k: v.clone() for k, v in st0.rhs_op.items()}
    op_sum = {k: torch.zeros_like(v) for k, v in op.items()}
    glob, glob_sum = glob0.clone(), torch.zeros(dim)
    it = iter(drawn)
    seen = {}
    for call in loop.calls_log:
        b, k, b_now = call["bucket"], call["workers"], call["batch_size"]
        lhs, rhs, rel = call["lhs"], call["rhs"], call["rel"]
        assert lhs.shape == (k * b_now,) and rel.shape == (k,) and k <= workers
        # a batch holds edges of its one relation type, taken from the bucket
        el, er, erel = edges[(b.lhs, b.rhs)]
        keys = set(zip(el.tolist(), er.tolist(), erel.tolist()))
        for i in range(k):
            for a, c in zip(lhs[i * b_now:(i + 1) * b_now].tolist(), rhs[i * b_now:(i + 1) * b_now].tolist()):
                assert (a, c, int(rel[i])) in keys
        seen[(call["epoch"], b.lhs, b.rhs)] = seen.get((call["epoch"], b.lhs, b.rhs), 0) + k * b_now
        st = ostep.make_state(cfg, w[b.lhs], None if b.lhs == b.rhs else w[b.rhs])
        st.g_lhs = g[b.lhs]
        st.g_rhs = g[b.lhs] if b.lhs == b.rhs else g[b.rhs]
        st.rhs_op, st.rhs_op_sum = op, op_sum
        st.glob_lhs = st.glob_rhs = glob  # one entity type: one vector, whatever the partitions
        st.glob_lhs_sum = st.glob_rhs_sum = glob_sum
        ul, ur = next(it), next(it)
        batches = [(lhs[i * b_now:(i + 1) * b_now], rhs[i * b_now:(i + 1) * b_now], int(rel[i]), ul[i], ur[i])
                   for i in range(k)]
        ostep.train_lockstep(cfg, st, batches)
    for (epoch, l, r), count in seen.items():
        assert count == edges[(l, r)][0].shape[0]
    assert len(seen) == 2 * nparts * nparts
    for p in range(nparts):
        assert torch.allclose(store.tables[("e", p)], w[p], rtol=1e-4, atol=1e-6)
    assert not torch.equal(glob, glob0)
    assert torch.allclose(glob_dev.cpu(), glob, rtol=1e-4, atol=1e-6)
    assert torch.allclose(glob_sum_dev.cpu(), glob_sum, rtol=1e-4, atol=1e-9)
    for k in op:
        assert not torch.equal(op[k], st0.rhs_op[k])
        assert torch.allclose(rhs_op[k].cpu(), op[k], rtol=1e-4, atol=1e-6)
        assert torch.allclose(rhs_sum[k].cpu(), op_sum[k], rtol=1e-4, atol=1e-9)

"""The lock-step call at the worker counts the benchmark and the bucket loop run
(K = 20, 64, 65, 256), against oracle.step.train_lockstep (K HOGWILD workers,
train_cpu.py:849-884, in the one deterministic interleaving) on reduced-entity
versions of the BASELINE configurations.

K selects code paths of its own: the width of the batch field in the sort keys,
the per-row search over a row's K runs in the RowAdagrad update
(row_adagrad.py:80-96 applied K times in order), the one-wave parameter update
for K <= 64 and the looped one above it, the 64-batch blocks of the global
embeddings' update, the splitting of a relation's runs into ceil(64 / K) parts
for per-edge `linear` operators.  The entity counts are small so that every row
is named by many of the K batches, and relation counts are small so that
several batches of a call share a relation."""
import pytest
import torch

from oracle import step as ostep
from tests.parity import Census, anchored_state, double_state, adagrad_noise_slack, hinge_tie_rows, violator_ties, zipf_ids
from tests.test_gpu_step import pack, say, to_runner

pytestmark = pytest.mark.gpu

CASES = {
    # cfg1: identity, dot, ranking, dim 100, 50 + 50 negatives, embeddings N(0, 1e-3)
    "cfg1": dict(operator="none", comparator="dot", loss="ranking", dim=100, num_pos=1000, num_batch_negs=50,
                 num_uniform_negs=50, entities=5000, scale=1e-3, ks=(20, 64, 65, 256)),
    # ... with embeddings of size 0.3, where about half of the hinges are inactive
    "cfg1-trained": dict(operator="none", comparator="dot", loss="ranking", dim=100, num_pos=400, num_batch_negs=50,
                         num_uniform_negs=50, entities=5000, scale=0.03, ks=(64,)),
    # cfg4: translation, l2, ranking, dim 100, two tables, Zipf(1.8) ids: one entity on about 40 % of a side's edges
    "cfg4": dict(operator="translation", comparator="l2", loss="ranking", dim=100, num_pos=1000, num_batch_negs=50,
                 num_uniform_negs=50, entities=20000, scale=1e-3, zipf=1.8, shared=False, ks=(20, 64, 65, 256)),
    "cfg4-trained": dict(operator="translation", comparator="l2", loss="ranking", dim=100, num_pos=400, num_batch_negs=50,
                         num_uniform_negs=50, entities=20000, scale=0.1, zipf=1.8, shared=False, ks=(64,)),
    # cfg2: complex_diagonal, dot, softmax, dim 400, wide negative sets, Zipf(1.1) entities and relations
    "cfg2": dict(operator="complex_diagonal", comparator="dot", loss="softmax", dim=400, num_pos=200, num_batch_negs=50,
                 num_uniform_negs=300, entities=3000, relations=12, scale=0.1, zipf=1.1, rel_zipf=1.1, ks=(20, 64, 65, 256)),
    # ... with one relation per edge, at a dim the streaming kernels take (the run's parameter gradient and the
    # relation's K Adagrad steps come from two kernels of their own there)
    "cfg2-dynamic-dim256": dict(operator="complex_diagonal", comparator="dot", loss="softmax", dim=256, num_pos=200,
                                dynamic=True, num_batch_negs=50, num_uniform_negs=100, entities=3000, relations=12, scale=0.1,
                                zipf=1.1, rel_zipf=1.1, ks=(20, 64, 65)),
    "cfg2-dynamic": dict(operator="complex_diagonal", comparator="dot", loss="softmax", dim=64, num_pos=200, dynamic=True,
                         num_batch_negs=50, num_uniform_negs=100, entities=3000, relations=12, scale=0.1, zipf=1.1,
                         rel_zipf=1.1, ks=(20, 65)),
    # cfg5: linear, cos, logistic, one relation per edge, batches sorted by relation, Zipf(1.2) relations
    "cfg5": dict(operator="linear", comparator="cos", loss="logistic", dim=64, num_pos=400, dynamic=True,
                 num_batch_negs=100, num_uniform_negs=100, entities=4000, relations=12, scale=0.3, rel_zipf=1.2,
                 ks=(20, 64, 65)),
    "cfg5-dim256": dict(operator="linear", comparator="cos", loss="logistic", dim=256, num_pos=200, dynamic=True,
                        num_batch_negs=100, num_uniform_negs=100, entities=3000, relations=6, scale=0.3, rel_zipf=1.2,
                        ks=(20,)),
    "cfg5-standard": dict(operator="linear", comparator="cos", loss="logistic", dim=64, num_pos=200, num_batch_negs=100,
                          num_uniform_negs=100, entities=3000, relations=5, scale=0.3, ks=(20, 65)),
    # the element-wise operators with several batches per relation (one wave walks a parameter's K updates)
    "diagonal": dict(operator="diagonal", comparator="dot", loss="logistic", dim=32, num_pos=100, num_batch_negs=20,
                     num_uniform_negs=20, entities=1500, relations=5, scale=0.3, ks=(20, 64, 65)),
    "translation": dict(operator="translation", comparator="cos", loss="softmax", dim=32, num_pos=100, num_batch_negs=20,
                        num_uniform_negs=20, entities=1500, relations=5, scale=0.3, ks=(20, 64, 65)),
    "complex_diagonal": dict(operator="complex_diagonal", comparator="dot", loss="logistic", dim=32, num_pos=100,
                             num_batch_negs=20, num_uniform_negs=20, entities=1500, relations=5, scale=0.3, ks=(64, 65)),
    "affine": dict(operator="affine", comparator="dot", loss="logistic", dim=24, num_pos=100, num_batch_negs=20,
                   num_uniform_negs=20, entities=1500, relations=5, scale=0.3, ks=(20, 65)),
    "affine-dynamic": dict(operator="affine", comparator="cos", loss="logistic", dim=24, num_pos=100, dynamic=True,
                           num_batch_negs=20, num_uniform_negs=20, entities=1500, relations=5, scale=0.3, ks=(20, 65)),
    "diagonal-dynamic": dict(operator="diagonal", comparator="dot", loss="logistic", dim=32, num_pos=100, dynamic=True,
                             num_batch_negs=20, num_uniform_negs=20, entities=1500, relations=5, scale=0.3, ks=(64, 65)),
    # `linear` on rows wider than 1024 floats: every output coordinate sums that many products (the float64 anchor
    # and the Adagrad slack of this file's criterion are for exactly such sums)
    "linear-dim1536-dynamic": dict(operator="linear", comparator="dot", loss="logistic", dim=1536, num_pos=24, dynamic=True,
                                   num_batch_negs=8, num_uniform_negs=5, entities=300, relations=3, scale=0.03, ks=(1, 3)),
    "linear-dim1100": dict(operator="linear", comparator="cos", loss="softmax", dim=1100, num_pos=24, num_batch_negs=8,
                           num_uniform_negs=5, entities=300, relations=3, scale=0.03, ks=(1, 3)),
    "affine-dim2048": dict(operator="affine", comparator="l2", loss="ranking", dim=2048, num_pos=24, num_batch_negs=8,
                           num_uniform_negs=5, entities=300, relations=2, scale=0.03, shared=False, ks=(2,)),
    # rows wider than LDS (the chunk kernel on slices of 128 columns), power-law ids: the LiveJournal example's kind of step
    "sliced-cos": dict(operator="none", comparator="cos", loss="ranking", dim=256, num_pos=200, num_batch_negs=50,
                       num_uniform_negs=50, entities=3000, scale=0.1, zipf=1.5, ks=(20, 65)),
    "sliced-transe": dict(operator="translation", comparator="l2", loss="ranking", dim=200, num_pos=200, num_batch_negs=50,
                          num_uniform_negs=50, entities=20000, relations=4, scale=0.1, zipf=1.5, shared=False, ks=(64,)),
    # a table of 40 rows under a power law: the update takes a wave per table row, and the hot rows' runs are
    # hundreds of sorted positions long (many windows of 64 positions per run)
    "hot-row-walk": dict(operator="none", comparator="dot", loss="logistic", dim=100, num_pos=400, num_batch_negs=50,
                         num_uniform_negs=50, entities=40, scale=0.1, zipf=1.5, ks=(8, 20)),
    "hot-row-walk-wide": dict(operator="diagonal", comparator="cos", loss="softmax", dim=256, num_pos=300, num_batch_negs=50,
                              num_uniform_negs=50, entities=25, relations=3, scale=0.1, zipf=1.3, shared=False, ks=(5,)),
    # global embeddings: their update walks the batches in blocks of 64
    "global-fused": dict(operator="none", comparator="dot", loss="logistic", dim=100, num_pos=200, num_batch_negs=50,
                         num_uniform_negs=50, entities=3000, scale=0.1, global_emb=True, ks=(64, 65, 130)),
    "global-staged": dict(operator="diagonal", comparator="cos", loss="logistic", dim=32, num_pos=100, num_batch_negs=20,
                          num_uniform_negs=20, entities=1500, relations=5, scale=0.3, global_emb=True, shared=False,
                          ks=(20, 130)),
    # N3 regularizer at the FB15k example's setting
    "n3": dict(operator="complex_diagonal", comparator="dot", loss="softmax", dim=64, num_pos=100, num_batch_negs=50,
               num_uniform_negs=50, entities=1500, relations=5, scale=0.3, regularization_coef=1e-3, ks=(20, 65)),
}


def build(name, workers, seed):
    w = dict(CASES[name])
    w.pop("ks")
    num_pos, ents, scale = w.pop("num_pos"), w.pop("entities"), w.pop("scale")
    rels, zipf, rel_zipf = w.pop("relations", 1), w.pop("zipf", None), w.pop("rel_zipf", None)
    shared = w.pop("shared", True)
    g = torch.Generator().manual_seed(seed)
    cfg = ostep.StepConfig(num_relations=rels, relation_weights=[1.0 + 0.25 * (r % 3) for r in range(rels)], lr=0.1,
                           relation_lr=0.01, margin=0.1, **w)
    _, c, _ = cfg.chunking(num_pos)
    u = cfg.num_uniform_negs
    w_l = torch.randn(ents, cfg.dim, generator=g) * scale
    w_r = None if shared else torch.randn(ents + 5, cfg.dim, generator=g) * scale
    n_r = ents if shared else ents + 5

    def draw(n, num):
        return zipf_ids(n, num, zipf, g) if zipf else torch.randint(0, num, (n,), generator=g)

    batches = []
    for _ in range(workers):
        lhs, rhs = draw(num_pos, ents), draw(num_pos, n_r)
        ul = torch.randint(0, ents, (c, u), generator=g)
        ur = torch.randint(0, n_r, (c, u), generator=g)
        if cfg.dynamic:
            rel = zipf_ids(num_pos, rels, rel_zipf, g) if rel_zipf else torch.randint(0, rels, (num_pos,), generator=g)
            rel = rel.sort().values  # mixed batches sorted by relation
        else:
            rel = int(zipf_ids(1, rels, rel_zipf, g)) if rel_zipf else int(torch.randint(0, rels, (1,), generator=g))
        batches.append((lhs, rhs, rel, ul, ur))
    st = ostep.make_state(cfg, w_l, w_r)
    for d in (st.lhs_op, st.rhs_op):
        for k in d:
            d[k] = d[k] + 0.1 * torch.randn(d[k].shape, generator=g)
    if st.glob_lhs is not None:
        st.glob_lhs += 0.3 * scale * torch.randn(cfg.dim, generator=g)
        if st.glob_rhs is not st.glob_lhs:
            st.glob_rhs += 0.3 * scale * torch.randn(cfg.dim, generator=g)
    return cfg, st, batches, num_pos


PARAMS = [(name, k) for name in CASES for k in CASES[name]["ks"]]


@pytest.mark.parametrize("name,workers", PARAMS, ids=[f"{n}-K{k}" for n, k in PARAMS])
def test_many_workers_match_the_lockstep_oracle(pbg, name, workers):
    say("many workers", name, workers)
    cfg, st, batches, num_pos = build(name, workers, seed=1000 * workers)
    st64 = double_state(st)
    # A hinge argument within rounding distance of 0 may fall on either side in two
    # correct fp32 evaluations.  The rows such a tie reaches are held to "moved by at
    # most the steps a tie can flip", and so are the operator parameters of a call
    # with ties (an Adagrad step never exceeds the step size); everything else to 1e-5.
    tied = ([], [])
    tied_batches = 0
    if cfg.loss == "ranking":
        for b in batches:
            sc = ostep.forward_backward(cfg, st64, *b, keep_scores=True)[0].scores
            rows = hinge_tie_rows(cfg, sc, b[0], b[1], b[3], b[4])
            tied_batches += bool(rows[0] or rows[1])
            tied[0].extend(rows[0])
            tied[1].extend(rows[1])
        say("  batches with hinge ties", tied_batches, "rows reached", len(set(tied[0])) + len(set(tied[1])))
        assert tied_batches <= workers // 4 and len(tied[0]) + len(tied[1]) <= 200, "too many ties to say anything"
    # exact operator-parameter gradients of every batch (all batches read the state as it is on entry)
    grads64 = [ostep.forward_backward(cfg, st64, *b)[1] for b in batches] if (st.rhs_op or st.lhs_op) else []
    rel_lr = cfg.relation_lr if cfg.relation_lr is not None else cfg.lr
    slack = {side: {k: adagrad_noise_slack([getattr(g, side)[k] for g in grads64], rel_lr) for k in getattr(st, side)}
             for side in ("rhs_op", "lhs_op")} if grads64 else None
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs = ostep.train_lockstep(cfg, st, batches, keep_scores=True)
    ostep.train_lockstep(cfg, st64, batches)
    for k, out in enumerate(outs):
        assert float(runner.loss_out[k]) == pytest.approx(out.loss, rel=1e-5, abs=1e-6), ("loss", k)
        if cfg.regularization_coef:
            assert float(runner.reg_out[k]) == pytest.approx(out.reg, rel=1e-5), ("reg", k)
        sc = out.scores
        for side, pos, neg, want in ((0, sc.lhs_pos, sc.lhs_neg, out.violators_lhs),
                                     (1, sc.rhs_pos, sc.rhs_neg, out.violators_rhs)):
            ties = violator_ties(pos, neg)
            assert abs(int(runner.violators_out[k, side]) - want) <= ties, ("violators", side, k, ties)
    census = Census()
    loose_rows = None
    if tied_batches:
        loose_rows = [torch.zeros(st.w_lhs.shape[0], dtype=torch.bool), torch.zeros(st.w_rhs.shape[0], dtype=torch.bool)]
        loose_rows[0][torch.tensor(tied[0], dtype=torch.int64)] = True
        loose_rows[1][torch.tensor(tied[1], dtype=torch.int64)] = True
        if st.shared:
            loose_rows[0] |= loose_rows[1]
            loose_rows[1] = loose_rows[0]
    anchored_state(cfg, runner, st, st64, 1e-5, f"{name} K={workers}", census, loose_rows=loose_rows,
                   loose_steps=2 * tied_batches, param_slack=slack)
    say("  ", census)
    # the float64 anchor is for the odd entry whose fp32 sum depends on the order of summation,
    # not a second criterion that everything may pass on
    assert census.anchored <= max(5, 1e-4 * census.entries), str(census)

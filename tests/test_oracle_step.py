"""Pins the parts of the oracle the reference's own tests leave open:
chunking / negatives / masks (against the independent per-edge float64 brute
force and closed-form invariants), the losses (textbook forms), RowAdagrad and
AsyncAdagrad (reductions to torch.optim.Adagrad, duplicate handling)."""
import itertools

import numpy as np
import pytest
import torch

from oracle import brute, step


def make_case(cfg, num_pos, n_ent, seed, shared=True, scale=0.5):
    g = torch.Generator().manual_seed(seed)
    w_l = torch.randn(n_ent, cfg.dim, generator=g) * scale
    w_r = w_l if shared else torch.randn(n_ent + 3, cfg.dim, generator=g) * scale
    lhs = torch.randint(0, w_l.shape[0], (num_pos,), generator=g)
    rhs = torch.randint(0, w_r.shape[0], (num_pos,), generator=g)
    _, c, _ = cfg.chunking(num_pos)
    u = cfg.num_uniform_negs
    ul = torch.randint(0, w_l.shape[0], (c, u), generator=g)
    ur = torch.randint(0, w_r.shape[0], (c, u), generator=g)
    rel = torch.randint(0, cfg.num_relations, (num_pos,), generator=g) if cfg.dynamic else int(
        torch.randint(0, cfg.num_relations, (1,), generator=g))
    st = step.make_state(cfg, w_l, None if shared else w_r)
    for d in (st.lhs_op, st.rhs_op):
        for k in d:
            d[k] = d[k] + 0.3 * torch.randn(d[k].shape, generator=g)
    return st, lhs, rhs, rel, ul, ur


def run_forward(cfg, st, lhs, rhs, rel, ul, ur):
    lp, rp = st.w_lhs[lhs], st.w_rhs[rhs]
    if cfg.all_negs:
        lu = None if cfg.disable_lhs_negs else st.w_lhs.unsqueeze(0)
        ru = None if cfg.disable_rhs_negs else st.w_rhs.unsqueeze(0)
        return step.model_forward(cfg, lp, rp, lu, ru, rel, st.lhs_op or None, st.rhs_op or None, lhs_ids=lhs, rhs_ids=rhs)
    lu = st.w_lhs[ul] if (cfg.num_uniform_negs > 0 and not cfg.disable_lhs_negs) else None
    ru = st.w_rhs[ur] if (cfg.num_uniform_negs > 0 and not cfg.disable_rhs_negs) else None
    return step.model_forward(cfg, lp, rp, lu, ru, rel, st.lhs_op or None, st.rhs_op or None)


CASES = []
for op, cmp_, dyn in itertools.product(step.OPERATOR_NAMES, step.COMPARATOR_NAMES, (False, True)):
    CASES.append(dict(operator=op, comparator=cmp_, dynamic=dyn, num_batch_negs=4, num_uniform_negs=3, num_pos=10))
CASES += [
    dict(operator="diagonal", comparator="dot", dynamic=False, num_batch_negs=4, num_uniform_negs=0, num_pos=8),
    dict(operator="diagonal", comparator="dot", dynamic=False, num_batch_negs=0, num_uniform_negs=3, num_pos=7),
    dict(operator="translation", comparator="l2", dynamic=True, num_batch_negs=0, num_uniform_negs=5, num_pos=3),
    dict(operator="none", comparator="cos", dynamic=False, num_batch_negs=16, num_uniform_negs=2, num_pos=5),
    dict(operator="complex_diagonal", comparator="dot", dynamic=False, num_batch_negs=4, num_uniform_negs=3,
         num_pos=9, disable_lhs_negs=True),
    dict(operator="complex_diagonal", comparator="dot", dynamic=True, num_batch_negs=4, num_uniform_negs=3,
         num_pos=9, disable_rhs_negs=True),
    dict(operator="linear", comparator="cos", dynamic=False, num_batch_negs=3, num_uniform_negs=2, num_pos=7,
         shared=False),
]
# RelationSchema.all_negs (model.py:648-650,582-618), standard and dynamic, one table and two
for cmp_, dyn, sh in itertools.product(("dot", "l2"), (False, True), (True, False)):
    CASES.append(dict(operator="diagonal", comparator=cmp_, dynamic=dyn, num_batch_negs=4, num_uniform_negs=3, num_pos=10,
                      all_negs=True, shared=sh))
CASES.append(dict(operator="translation", comparator="cos", dynamic=False, num_batch_negs=0, num_uniform_negs=0, num_pos=7,
                  all_negs=True, disable_lhs_negs=True))
# config.bias (BiasedComparator, model.py:306-344) around every comparator, standard and dynamic
for cmp_, dyn in itertools.product(step.COMPARATOR_NAMES, (False, True)):
    CASES.append(dict(operator="diagonal" if dyn else "translation", comparator=cmp_, dynamic=dyn, num_batch_negs=4,
                      num_uniform_negs=3, num_pos=10, bias=True))


@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(str(v) for v in c.values()))
def test_forward_matches_brute_force(case):
    case = dict(case)
    num_pos = case.pop("num_pos")
    shared = case.pop("shared", True)
    cfg = step.StepConfig(dim=6, num_relations=3, relation_weights=[1.0, 1.0, 1.0], **case)
    st, lhs, rhs, rel, ul, ur = make_case(cfg, num_pos, 11, seed=num_pos, shared=shared)
    s = run_forward(cfg, st, lhs, rhs, rel, ul, ur)
    blp, brp, bln, brn = brute.scores(
        cfg, st.w_lhs.numpy(), st.w_rhs.numpy(), lhs.numpy(), rhs.numpy(),
        rel if isinstance(rel, int) else rel.numpy(), ul.numpy(), ur.numpy(),
        {k: v.numpy() for k, v in st.lhs_op.items()}, {k: v.numpy() for k, v in st.rhs_op.items()})
    for got, want in ((s.lhs_pos, blp), (s.rhs_pos, brp), (s.lhs_neg, bln), (s.rhs_neg, brn)):
        assert tuple(got.shape) == want.shape
        got = got.numpy().astype(np.float64)
        if cfg.comparator == "l2":
            # the reference's ||a||^2 - 2ab + ||b||^2 expansion cancels badly at
            # (near-)zero distance: compare squared distances there
            live = want != -1e9
            np.testing.assert_allclose(got[live] ** 2, want[live] ** 2, rtol=2e-5, atol=2e-5)
            assert (got[~live] == -1e9).all()
        else:
            np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)
    # masked entries are exactly -1e9
    assert ((s.lhs_neg == -1e9).numpy() == (bln == -1e9)).all()
    assert ((s.rhs_neg == -1e9).numpy() == (brn == -1e9)).all()
    for name in step.LOSS_NAMES:
        for pos, neg, bp, bn in ((s.lhs_pos, s.lhs_neg, blp, bln), (s.rhs_pos, s.rhs_neg, brp, brn)):
            got = float(step.loss_value(name, pos, neg, None, margin=0.1))
            want = brute.loss(name, pos.double().numpy(), neg.double().numpy(), 0.1)
            assert got == pytest.approx(want, rel=1e-5, abs=1e-5)


@pytest.mark.parametrize("comparator", step.COMPARATOR_NAMES)
@pytest.mark.parametrize("dynamic", [False, True])
def test_bias_reduces_to_the_base_comparator_and_shifts_scores(comparator, dynamic):
    """What the definition of BiasedComparator fixes (model.py:306-344), without
    the brute force: (1) with a zero first coordinate everywhere, and an operator
    that keeps it zero, the scores are the base comparator's on the remaining
    D - 1 coordinates -- which the reference's own vectors pin; (2) adding c to
    every row's first coordinate adds 2c to every score that is not masked."""
    kw = dict(operator="diagonal", comparator=comparator, dynamic=dynamic, num_batch_negs=4, num_uniform_negs=3,
              num_relations=3, relation_weights=[1.0, 1.0, 1.0])
    cfg_b = step.StepConfig(dim=6, bias=True, **kw)
    cfg_0 = step.StepConfig(dim=5, **kw)
    st, lhs, rhs, rel, ul, ur = make_case(cfg_b, 10, 11, seed=5)
    st.w_lhs[:, 0] = 0.0
    st.w_rhs[:, 0] = 0.0
    s_b = run_forward(cfg_b, st, lhs, rhs, rel, ul, ur)
    st0 = step.make_state(cfg_0, st.w_lhs[:, 1:].clone(), None if st.shared else st.w_rhs[:, 1:].clone())
    st0.lhs_op = {k: v[:, 1:].clone() for k, v in st.lhs_op.items()}
    st0.rhs_op = {k: v[:, 1:].clone() for k, v in st.rhs_op.items()}
    s_0 = run_forward(cfg_0, st0, lhs, rhs, rel, ul, ur)
    for a, b in zip((s_b.lhs_pos, s_b.rhs_pos, s_b.lhs_neg, s_b.rhs_neg), (s_0.lhs_pos, s_0.rhs_pos, s_0.lhs_neg, s_0.rhs_neg)):
        assert torch.allclose(a, b, rtol=1e-6, atol=1e-6)
    # (2): the diagonal operator scales the first coordinate of the operated rows; with 1 there the shift is c + c
    for d in (st.lhs_op, st.rhs_op):
        for v in d.values():
            v[:, 0] = 1.0
    base = run_forward(cfg_b, st, lhs, rhs, rel, ul, ur)
    st.w_lhs[:, 0] += 0.25
    if not st.shared:
        st.w_rhs[:, 0] += 0.25
    moved = run_forward(cfg_b, st, lhs, rhs, rel, ul, ur)
    for a, b in zip((base.lhs_pos, base.rhs_pos, base.lhs_neg, base.rhs_neg),
                    (moved.lhs_pos, moved.rhs_pos, moved.lhs_neg, moved.rhs_neg)):
        live = a != -1e9
        assert torch.equal(b == -1e9, ~live)
        assert torch.allclose(b[live], a[live] + 0.5, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dynamic", [False, True])
def test_all_negs_is_uniform_mode_over_every_entity_with_the_own_entity_masked(dynamic):
    """all_negs reduces to a path the other tests pin: uniform-only negatives
    (model.py:651-653) with U = E "samples" 0 .. E-1 in one chunk give the same
    scores, except that all_negs masks column lhs[i] (rhs[i]) of row i."""
    kw = dict(dim=6, operator="diagonal", comparator="cos", dynamic=dynamic, num_relations=3, relation_weights=[1.0] * 3)
    n_ent, num_pos = 13, 9
    cfg_all = step.StepConfig(all_negs=True, num_batch_negs=5, num_uniform_negs=2, **kw)
    cfg_uni = step.StepConfig(num_batch_negs=0, num_uniform_negs=n_ent, **kw)  # chunk = min(U, B) = B: one chunk
    st, lhs, rhs, rel, _, _ = make_case(cfg_all, num_pos, n_ent, seed=2)
    every = torch.arange(n_ent).unsqueeze(0)
    a = run_forward(cfg_all, st, lhs, rhs, rel, None, None)
    u = run_forward(cfg_uni, st, lhs, rhs, rel, every, every)
    assert torch.equal(a.lhs_pos, u.lhs_pos) and torch.equal(a.rhs_pos, u.rhs_pos)
    for got, want, ids in ((a.lhs_neg, u.lhs_neg, lhs), (a.rhs_neg, u.rhs_neg, rhs)):
        own = torch.zeros_like(got, dtype=torch.bool)
        own[torch.arange(num_pos), ids] = True
        assert torch.equal(got == -1e9, own)
        assert torch.equal(got[~own], want[~own])


def test_invariants_single_chunk_no_uniform():
    """U = 0, C = 1, identity + dot: lhs_neg = R L^T, rhs_neg = L R^T off the
    diagonal, and pos is their common pre-mask diagonal."""
    cfg = step.StepConfig(dim=5, num_batch_negs=6, num_uniform_negs=0)
    st, lhs, rhs, rel, ul, ur = make_case(cfg, 6, 9, seed=3)
    s = run_forward(cfg, st, lhs, rhs, rel, ul, ur)
    l, r = st.w_lhs[lhs], st.w_rhs[rhs]
    full_l, full_r = r @ l.T, l @ r.T
    off = ~torch.eye(6, dtype=torch.bool)
    assert torch.allclose(s.lhs_neg[off], full_l[off], atol=1e-6)
    assert torch.allclose(s.rhs_neg[off], full_r[off], atol=1e-6)
    assert torch.allclose(s.lhs_pos, full_l.diagonal(), atol=1e-6)
    assert (s.lhs_neg.diagonal() == -1e9).all() and (s.rhs_neg.diagonal() == -1e9).all()


def test_ranking_subgradient_at_the_hinge():
    """torch's hinge passes the gradient where margin - s + t is exactly 0."""
    pos = torch.tensor([1.0], requires_grad=True)
    neg = torch.tensor([[0.5, 0.25, 0.75]], requires_grad=True)
    step.loss_value("ranking", pos, neg, None, margin=0.5).backward()
    assert neg.grad.tolist() == [[1.0, 0.0, 1.0]]
    assert pos.grad.tolist() == [-2.0]


def test_row_adagrad_reduces_to_adagrad():
    """(a) dim 1 and (b) rows whose gradient entries are all equal make the
    row-wise mean of g^2 equal the element-wise g^2, so RowAdagrad must agree
    with torch.optim.Adagrad(eps=1e-10) -- a sum instead of a mean, a missing
    sqrt or a wrong sign all break this."""
    for dim in (1, 4):
        torch.manual_seed(dim)
        w = torch.randn(7, dim)
        ref = torch.nn.Parameter(w.clone())
        opt = torch.optim.Adagrad([ref], lr=0.1, eps=1e-10)
        mine, gsum = w.clone(), torch.zeros(7)
        for it in range(5):
            idx = torch.tensor([1, 3, 6]) if it % 2 == 0 else torch.tensor([0, 3])
            vals = torch.randn(len(idx), 1).expand(len(idx), dim).contiguous()
            dense = torch.zeros(7, dim).index_add_(0, idx, vals)
            opt.zero_grad()
            ref.grad = dense.clone()
            opt.step()
            sp = torch.sparse_coo_tensor(idx.unsqueeze(0), vals, (7, dim))
            step.row_adagrad_sparse(mine, gsum, sp, 0.1)
        assert torch.allclose(mine, ref.detach(), rtol=1e-6, atol=1e-7)


def test_row_adagrad_duplicates_and_monotone_state():
    torch.manual_seed(0)
    w = torch.randn(5, 3)
    idx = torch.tensor([2, 4, 2, 2, 0])
    vals = torch.randn(5, 3)
    a, ga = w.clone(), torch.full((5,), 0.25)
    step.row_adagrad_sparse(a, ga, torch.sparse_coo_tensor(idx.unsqueeze(0), vals, (5, 3)), 0.05)
    # pre-summed by hand
    uniq = torch.tensor([0, 2, 4])
    summed = torch.stack([vals[4], vals[0] + vals[2] + vals[3], vals[1]])
    b, gb = w.clone(), torch.full((5,), 0.25)
    for r, g in zip(uniq.tolist(), summed):
        delta = float((g.double() ** 2).mean())
        b[r] -= 0.05 * g / (np.sqrt(0.25 + delta) + 1e-10)
        gb[r] += delta
    assert torch.allclose(a, b, rtol=1e-6, atol=1e-7)
    assert torch.allclose(ga, gb, rtol=1e-6)
    assert (ga >= 0.25).all() and torch.equal(a[[1, 3]], w[[1, 3]])
    # dense branch agrees with the sparse branch on the same gradient
    c, gc = w.clone(), torch.full((5,), 0.25)
    dense = torch.zeros(5, 3).index_add_(0, idx, vals)
    step.row_adagrad_dense(c, gc, dense, 0.05)
    assert torch.allclose(a, c, rtol=1e-6, atol=1e-7) and torch.allclose(ga, gc, rtol=1e-6)
    # empty gradient is a no-op
    step.row_adagrad_sparse(a, ga, torch.sparse_coo_tensor(torch.empty(1, 0, dtype=torch.long), torch.empty(0, 3), (5, 3)), 0.05)
    assert torch.allclose(a, c, rtol=1e-6, atol=1e-7)


def test_async_adagrad_equals_adagrad():
    """The reference's own claim (test/test_optimizers.py:110-130)."""
    torch.manual_seed(1)
    p0 = torch.randn(4, 6)
    ref = torch.nn.Parameter(p0.clone())
    opt = torch.optim.Adagrad([ref], lr=0.01, eps=1e-10)
    mine, gsum = p0.clone(), torch.zeros(4, 6)
    for _ in range(6):
        g = torch.randn(4, 6)
        ref.grad = g.clone()
        opt.step()
        step.async_adagrad_dense(mine, gsum, g, 0.01)
    assert torch.allclose(mine, ref.detach(), rtol=1e-6, atol=1e-7)


def test_backward_matches_finite_differences():
    """Autograd through the oracle forward against central differences in
    float64, for the comparator with the trickiest derivative (l2) and an
    operator with parameters."""
    cfg = step.StepConfig(dim=4, operator="complex_diagonal", comparator="l2", loss="softmax",
                          num_batch_negs=3, num_uniform_negs=2)
    st, lhs, rhs, rel, ul, ur = make_case(cfg, 5, 40, seed=5)
    # distinct entities everywhere: l2 has a kink at zero distance
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(0))
    lhs, rhs, ul, ur = perm[:5], perm[5:10], perm[10:14].view(2, 2), perm[14:18].view(2, 2)
    w = st.w_lhs.double()
    params = {k: v.double() for k, v in st.rhs_op.items()}

    def f(wt, real):
        p = dict(params, real=real)
        s = step.model_forward(cfg, wt[lhs], wt[rhs], wt[ul], wt[ur], rel, None, p)
        return (step.loss_value("softmax", s.lhs_pos, s.lhs_neg, None)
                + step.loss_value("softmax", s.rhs_pos, s.rhs_neg, None))

    assert torch.autograd.gradcheck(f, (w.requires_grad_(True), params["real"].requires_grad_(True)),
                                    eps=1e-6, atol=1e-5)


def test_lockstep_with_one_worker_is_the_sequential_step():
    cfg = step.StepConfig(dim=6, operator="translation", comparator="l2", loss="ranking",
                          num_batch_negs=4, num_uniform_negs=3)
    st_a, lhs, rhs, rel, ul, ur = make_case(cfg, 8, 12, seed=7)
    st_b, *_ = make_case(cfg, 8, 12, seed=7)
    step.train_step(cfg, st_a, lhs, rhs, rel, ul, ur)
    step.train_lockstep(cfg, st_b, [(lhs, rhs, rel, ul, ur)])
    assert torch.equal(st_a.w_lhs, st_b.w_lhs) and torch.equal(st_a.g_lhs, st_b.g_lhs)
    assert torch.equal(st_a.rhs_op["translation"], st_b.rhs_op["translation"])
    assert (st_a.g_lhs > 0).any()

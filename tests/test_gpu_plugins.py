"""GPU parity of the plugin classes (operators, comparators, losses, model,
optimizers, trainer, _C): the reference's own literal test vectors replayed
through the GPU classes, and forward / backward against the CPU oracle."""
import itertools

import numpy as np
import pytest
import torch

from oracle import perm as operm
from oracle import step as ostep

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PLURAL = {"diagonals": "diagonal", "translations": "translation", "linear_transformations": "linear_transformation"}


def say(*a):
    print(*a, flush=True)


def close(a, b, tol):
    return torch.allclose(a.detach().cpu(), torch.as_tensor(b, dtype=torch.float32), rtol=tol, atol=tol, equal_nan=True)


def test_reference_operator_vectors(pbg, golden):
    tol = golden["tolerance"]
    for case in golden["operators"]:
        say("operator", case["name"], case["dynamic"])
        x = torch.tensor(case["input"], device=DEV, requires_grad=True)
        if case["dynamic"]:
            op = pbg.operators.DYNAMIC_OPERATORS.get_class(case["name"])(case["dim"], case["num_operations"]).to(DEV)
        else:
            op = pbg.operators.OPERATORS.get_class(case["name"])(case["dim"]).to(DEV)
        with torch.no_grad():
            for k, v in case["params"].items():
                getattr(op, k)[...] = torch.tensor(v, device=DEV)
        y = op(x, torch.tensor(case["rel"], device=DEV)) if case["dynamic"] else op(x)
        assert y.shape == x.shape
        assert close(y, case["expected"], tol), (case["name"], case["dynamic"])
        y.sum().backward()
        assert (x.grad != 0).any()
        for p in op.parameters():
            assert (p.grad != 0).any()
        # gradients against autograd through the oracle
        xo = torch.tensor(case["input"], requires_grad=True)
        po = {PLURAL.get(k, k): torch.tensor(v).requires_grad_(True) for k, v in case["params"].items()}
        if not case["dynamic"]:
            po = {k: v.detach().unsqueeze(0).requires_grad_(True) for k, v in po.items()}
        ostep.apply_operator(case["name"], xo, po, torch.tensor(case["rel"]) if case["dynamic"] else 0).sum().backward()
        assert close(x.grad, xo.grad, 1e-5)
        for k in case["params"]:
            want = po[PLURAL.get(k, k)].grad
            assert close(getattr(op, k).grad, want if case["dynamic"] else want[0], 1e-5), k


def test_reference_comparator_vectors(pbg, golden):
    tol = golden["tolerance"]
    for case in golden["comparators"]:
        say("comparator", case["name"], case["ref"])
        cmp_ = pbg.model.COMPARATORS.get_class(case["name"])()
        ts = [torch.tensor(case[k], device=DEV, requires_grad=True) for k in ("lhs_pos", "rhs_pos", "lhs_neg", "rhs_neg")]
        pos, lneg, rneg = cmp_(*[cmp_.prepare(t) for t in ts])
        assert close(pos, case["pos"], tol) and close(lneg, case["lhs_neg_scores"], tol) and close(rneg, case["rhs_neg_scores"], tol)
        (pos.sum() + lneg.sum() + rneg.sum()).backward()
        for t in ts:
            assert (t.grad != 0).any()


def test_reference_biased_comparator_vectors(pbg, golden):
    tol = golden["tolerance"]
    for case in golden["biased_comparators"]:
        say("biased comparator", case["name"], case["ref"])
        cmp_ = pbg.model.BiasedComparator(pbg.model.COMPARATORS.get_class(case["name"])())
        ts = [torch.tensor(case[k], device=DEV, requires_grad=True) for k in ("lhs_pos", "rhs_pos", "lhs_neg", "rhs_neg")]
        pos, lneg, rneg = cmp_(*[cmp_.prepare(t) for t in ts])
        assert close(pos, case["pos"], tol) and close(lneg, case["lhs_neg_scores"], tol) and close(rneg, case["rhs_neg_scores"], tol)
        (pos.sum() + lneg.sum() + rneg.sum()).backward()
        for t in ts:
            assert (t.grad != 0).any()


@pytest.mark.parametrize("name", ["dot", "cos", "l2", "squared_l2"])
@pytest.mark.parametrize("shape", [(3, 5, 7, 4, 6), (1, 50, 100, 100, 100), (2, 4, 0, 3, 8), (2, 100, 130, 70, 256)])
def test_comparator_forward_backward_vs_oracle(pbg, name, shape):
    say("comparator grad", name, shape)
    c, p, ln, rn, d = shape
    g = torch.Generator().manual_seed(sum(shape))
    raw = [torch.randn(c, n, d, generator=g) for n in (p, p, ln, rn)]
    weights = [torch.randn(c, p, generator=g), torch.randn(c, p, ln, generator=g), torch.randn(c, p, rn, generator=g)]
    cmp_ = pbg.model.COMPARATORS.get_class(name)()
    ts = [t.clone().to(DEV).requires_grad_(True) for t in raw]
    outs = cmp_(*[cmp_.prepare(t) for t in ts])
    sum((o * w.to(DEV)).sum() for o, w in zip(outs, weights)).backward()
    to = [t.clone().requires_grad_(True) for t in raw]
    oo = ostep.comparator_scores(name, *[ostep.comparator_prepare(name, t) for t in to])
    sum((o * w).sum() for o, w in zip(oo, weights)).backward()
    for got, want in zip(outs, oo):
        if name == "l2":
            assert torch.allclose(got.detach().cpu() ** 2, want.detach() ** 2, rtol=2e-5, atol=2e-5 * d)
        else:
            assert torch.allclose(got.detach().cpu(), want.detach(), rtol=1e-5, atol=1e-5 * d ** 0.5)
    for got, want in zip(ts, to):
        if want.numel() == 0:
            continue
        scale = want.grad.abs().max().item()
        assert torch.allclose(got.grad.cpu(), want.grad, rtol=1e-4, atol=2e-5 * max(scale, 1.0)), name


@pytest.mark.parametrize("name", ["dot", "cos", "squared_l2"])
def test_biased_comparator_forward_backward_vs_oracle(pbg, name):
    """BiasedComparator (model.py:306-344) around the package's comparators against
    the oracle's restatement, values and gradients."""
    say("biased comparator", name)
    c, p, ln, rn, d = 3, 5, 7, 4, 6
    g = torch.Generator().manual_seed(11)
    raw = [torch.randn(c, n, d, generator=g) for n in (p, p, ln, rn)]
    weights = [torch.randn(c, p, generator=g), torch.randn(c, p, ln, generator=g), torch.randn(c, p, rn, generator=g)]
    cmp_ = pbg.model.BiasedComparator(pbg.model.COMPARATORS.get_class(name)())
    ts = [t.clone().to(DEV).requires_grad_(True) for t in raw]
    outs = cmp_(*[cmp_.prepare(t) for t in ts])
    sum((o * w.to(DEV)).sum() for o, w in zip(outs, weights)).backward()
    to = [t.clone().requires_grad_(True) for t in raw]
    oo = ostep.biased_scores(name, *[ostep.biased_prepare(name, t) for t in to])
    sum((o * w).sum() for o, w in zip(oo, weights)).backward()
    for got, want in zip(outs, oo):
        assert torch.allclose(got.detach().cpu(), want.detach(), rtol=1e-5, atol=1e-5 * d ** 0.5)
    for got, want in zip(ts, to):
        assert torch.allclose(got.grad.cpu(), want.grad, rtol=1e-4, atol=2e-5 * max(want.grad.abs().max().item(), 1.0)), name


def test_reference_loss_vectors(pbg, golden):
    tol = golden["tolerance"]
    for case in golden["losses"]:
        say("loss", case["name"], case["case"])
        cls = pbg.losses.LOSS_FUNCTIONS.get_class(case["name"])
        fn = cls(margin=case["margin"] if case["margin"] is not None else 0.1)
        pos = torch.tensor(case["pos"], dtype=torch.float32, device=DEV, requires_grad=True)
        if "neg_shape" in case:
            neg = torch.empty(case["neg_shape"], device=DEV, requires_grad=True)
        else:
            neg = torch.tensor(case["neg"], dtype=torch.float32, device=DEV).view(len(case["pos"]), -1).requires_grad_(True)
        w = torch.tensor(case["weight"], device=DEV) if case["weight"] is not None else None
        loss = fn(pos, neg, w)
        assert loss.dim() == 0
        assert close(loss, case["expected"], tol), (case["name"], case["case"], float(loss))
        loss.backward()
        if case["case"] in ("forward", "weight_uniform", "weight_mixed"):
            po = torch.tensor(case["pos"], requires_grad=True)
            no = torch.tensor(case["neg"], requires_grad=True)
            wo = torch.tensor(case["weight"]) if case["weight"] is not None else None
            ostep.loss_value(case["name"], po, no, wo, case["margin"] or 0.1).backward()
            assert close(pos.grad, po.grad, 1e-5) and close(neg.grad, no.grad, 1e-5)


def test_gather_and_sampling(pbg, golden):
    g = golden["gather"]
    w = torch.nn.Parameter(torch.tensor(g["table"], device=DEV))
    emb = pbg.model.SimpleEmbedding(w)
    out = emb(pbg.entitylist.EntityList.from_tensor(torch.tensor(g["index"], device=DEV)))
    assert torch.equal(out.cpu(), torch.tensor(g["expected"]))
    out.sum().backward()
    assert w.grad.is_sparse and (w.grad.to_dense() != 0).any()
    assert torch.equal(emb.get_all_entities().detach().cpu(), torch.tensor(g["table"]))
    s = emb.sample_entities(2, 2)
    assert tuple(s.shape) == (2, 2, 3)
    empty = emb(pbg.entitylist.EntityList.from_tensor(torch.empty((0,), dtype=torch.long, device=DEV)))
    assert tuple(empty.shape) == (0, 3)
    # max_norm (test/test_model.py:72-84,102-116): looked-up rows are renormalised in the table first
    m = g["max_norm"]
    w = torch.nn.Parameter(torch.tensor(g["table"], device=DEV))
    emb = pbg.model.SimpleEmbedding(w, max_norm=m["max_norm"])
    out = emb(pbg.entitylist.EntityList.from_tensor(torch.tensor(m["index"], device=DEV)))
    assert close(out, m["expected"], golden["tolerance"])
    assert torch.equal(w.data[1].cpu(), torch.tensor(g["table"][1]))
    assert close(emb.get_all_entities(), m["all_entities_expected"], golden["tolerance"])
    assert close(w.data, m["all_entities_expected"], golden["tolerance"])
    assert float(emb.sample_entities(2, 2).detach().norm(dim=-1).max()) <= 2.0 * (1 + 1e-6)


def build_model(pbg, cfg, st, n_rel_schemas):
    O, M, C = pbg.operators, pbg.model, pbg.config
    dev = lambda t: torch.nn.Parameter(t.clone().to(DEV))
    w_l = dev(st.w_lhs)
    w_r = w_l if st.shared else dev(st.w_rhs)
    ent = {"l": C.EntitySchema(), "r": C.EntitySchema()}
    rels = [C.RelationSchema(name=f"r{i}", lhs="l", rhs="l" if st.shared else "r", operator=cfg.operator,
                             weight=cfg.relation_weights[i], all_negs=cfg.all_negs) for i in range(n_rel_schemas)]
    if cfg.dynamic:
        lhs_ops = [O.instantiate_operator(cfg.operator, pbg.types.Side.LHS, cfg.num_relations, cfg.dim).to(DEV)]
        rhs_ops = [O.instantiate_operator(cfg.operator, pbg.types.Side.RHS, cfg.num_relations, cfg.dim).to(DEV)]
    else:
        lhs_ops = [None] * n_rel_schemas
        rhs_ops = [O.instantiate_operator(cfg.operator, pbg.types.Side.RHS, 0, cfg.dim).to(DEV) for _ in range(n_rel_schemas)]
    names = {"diagonal": "diagonals", "translation": "translations", "linear_transformation": "linear_transformations"}
    with torch.no_grad():
        for ops, params in ((rhs_ops, st.rhs_op), (lhs_ops, st.lhs_op)):
            for k, v in params.items():
                if cfg.dynamic:
                    getattr(ops[0], names.get(k, k))[...] = v.to(DEV)
                else:
                    for i, op in enumerate(ops):
                        if op is not None:
                            getattr(op, k)[...] = v[i].to(DEV)
    regularizer = None
    if cfg.regularization_coef != 0:  # model.py:905-909
        regularizer = pbg.regularizers.REGULARIZERS.get_class("N3")(cfg.regularization_coef)
    comparator = M.COMPARATORS.get_class(cfg.comparator)()
    if cfg.bias:  # model.py:902-903
        comparator = M.BiasedComparator(comparator)
    model = M.MultiRelationEmbedder(
        cfg.dim, rels, ent, cfg.num_batch_negs, cfg.num_uniform_negs, cfg.disable_lhs_negs, cfg.disable_rhs_negs,
        lhs_ops, rhs_ops, comparator, regularizer=regularizer,
        global_emb=cfg.global_emb, max_norm=cfg.max_norm, num_dynamic_rels=cfg.num_relations if cfg.dynamic else 0,
        half_precision=cfg.half_precision)
    if cfg.global_emb:
        model.global_embs.to(DEV)
        with torch.no_grad():
            model.global_embs[M.MultiRelationEmbedder.EMB_PREFIX + "l"][...] = st.glob_lhs.to(DEV)
            if not st.shared:
                model.global_embs[M.MultiRelationEmbedder.EMB_PREFIX + "r"][...] = st.glob_rhs.to(DEV)
    model.set_embeddings("l", pbg.types.Side.LHS, w_l)
    model.set_embeddings("l" if st.shared else "r", pbg.types.Side.RHS, w_r)
    return model, w_l, w_r


MODEL_CASES = [
    dict(operator="none", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=100),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=10, num_uniform_negs=20, num_pos=40, dim=16),
    dict(operator="translation", comparator="l2", loss="ranking", dynamic=False, num_batch_negs=10, num_uniform_negs=10, num_pos=33, dim=12),
    dict(operator="linear", comparator="cos", loss="logistic", dynamic=False, num_batch_negs=8, num_uniform_negs=8, num_pos=24, dim=9),
    dict(operator="diagonal", comparator="cos", loss="logistic", dynamic=False, num_batch_negs=0, num_uniform_negs=7, num_pos=30, dim=9),
    # RelationSchema.all_negs: every entity of a side's type is a negative
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=10, num_uniform_negs=20,
         num_pos=40, dim=16, all_negs=True),
    dict(operator="diagonal", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=0, num_uniform_negs=0, num_pos=25,
         dim=9, all_negs=True),
    # config.bias: BiasedComparator around the comparator
    dict(operator="diagonal", comparator="cos", loss="ranking", dynamic=False, num_batch_negs=10, num_uniform_negs=20, num_pos=40,
         dim=16, bias=True),
    # (with one relation per edge the operated row's bias shifts every score of its row alike: under softmax the
    # operator's first element has a zero gradient, rounding noise for Adagrad -- logistic here)
    dict(operator="diagonal", comparator="dot", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=5, num_pos=25,
         dim=9, bias=True),
    # max_norm: about half of the rows (0.3 * randn, dim 16) are longer than 1.2
    dict(operator="diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=10, num_uniform_negs=20, num_pos=40,
         dim=16, max_norm=1.2),
    dict(operator="affine", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=8, num_uniform_negs=8, num_pos=24, dim=9),
    # rows wider than 1024 floats through the plugin classes
    dict(operator="complex_diagonal", comparator="cos", loss="softmax", dynamic=False, num_batch_negs=8, num_uniform_negs=8, num_pos=24, dim=2048),
    dict(operator="translation", comparator="l2", loss="ranking", dynamic=True, num_batch_negs=8, num_uniform_negs=8, num_pos=24, dim=4096),
    dict(operator="affine", comparator="l2", loss="softmax", dynamic=True, num_batch_negs=10, num_uniform_negs=5, num_pos=25, dim=8),
    dict(operator="none", comparator="dot", loss="softmax", dynamic=True, num_batch_negs=10, num_uniform_negs=5, num_pos=25, dim=8),
    # with the N3 regularizer (the reference's FB15k example uses 1e-3 on ComplEx)
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=10, num_uniform_negs=20,
         num_pos=45, dim=16, regularization_coef=1e-2),
    dict(operator="diagonal", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=5, num_pos=25,
         dim=8, regularization_coef=5e-2),
    dict(operator="translation", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=10, num_uniform_negs=5,
         num_pos=25, dim=9, regularization_coef=5e-2),
    # with global embeddings (the reference's default), one entity type (even dim) and two
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=10, num_uniform_negs=20,
         num_pos=45, dim=16, global_emb=True),
    dict(operator="diagonal", comparator="cos", loss="logistic", dynamic=False, num_batch_negs=10, num_uniform_negs=5,
         num_pos=25, dim=9, global_emb=True),
]


@pytest.mark.parametrize("case", MODEL_CASES, ids=lambda c: "-".join(str(v) for v in c.values()))
def test_model_forward_and_trainer_step(pbg, case):
    """MultiRelationEmbedder.forward and Trainer._process_one_batch (with
    RowAdagrad / AsyncAdagrad state owned by torch optimizers) against the oracle."""
    say("model", case)
    from tests.test_gpu_step import assert_close, compare_scores, make_inputs

    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, **case)
    st, batches = make_inputs(cfg, num_pos, 800 if cfg.comparator == "l2" else 300, 2, seed=dim, shared=(dim % 2 == 0))
    model, w_l, w_r = build_model(pbg, cfg, st, 1 if cfg.dynamic else 3)
    EL, ED = pbg.entitylist.EntityList, pbg.edgelist.EdgeList
    T = pbg.train
    loss_fn = pbg.losses.LOSS_FUNCTIONS.get_class(cfg.loss)(margin=cfg.margin)
    op_params = [p for p in model.parameters()]
    trainer = T.Trainer(T.make_optimizer(op_params, False, cfg.lr, cfg.relation_lr), loss_fn, list(cfg.relation_weights))
    trainer.partitioned_optimizers[("l", 0)] = T.make_optimizer([w_l], True, cfg.lr)
    if not st.shared:
        trainer.partitioned_optimizers[("r", 0)] = T.make_optimizer([w_r], True, cfg.lr)
    for lhs, rhs, rel, ul, ur in batches:
        rel_t = rel.to(DEV) if cfg.dynamic else torch.tensor(rel)
        edges = ED(EL.from_tensor(lhs.to(DEV)), EL.from_tensor(rhs.to(DEV)), rel_t)
        scores, reg = model(edges, uniform_negs=(ul.to(DEV), ur.to(DEV)))
        want, _ = ostep.forward_backward(cfg, st, lhs, rhs, rel, ul, ur, keep_scores=True)
        if cfg.regularization_coef == 0:
            assert reg is None
        else:
            assert float(reg) == pytest.approx(want.reg, rel=1e-5)
        compare_scores(cfg, tuple(scores), want.scores)
        trainer.next_uniform_negs = (ul.to(DEV), ur.to(DEV))
        stats = trainer.process_one_batch(model, edges)
        out = ostep.train_step(cfg, st, lhs, rhs, rel, ul, ur)
        rtol = 1e-4 if cfg.comparator == "l2" else 1e-5
        assert stats.count == num_pos
        assert stats.metrics["loss"] == pytest.approx(out.loss, rel=rtol, abs=1e-6)
        assert stats.metrics["reg"] == pytest.approx(out.reg, rel=1e-5)
        for side, pos, neg, n_want in (("lhs", want.scores.lhs_pos, want.scores.lhs_neg, out.violators_lhs),
                                       ("rhs", want.scores.rhs_pos, want.scores.rhs_neg, out.violators_rhs)):
            pp = pos.unsqueeze(1)
            ties = int(((neg - pp).abs() <= 2e-5 * pp.abs().clamp_min(1e-6)).sum())
            assert abs(stats.metrics["violators_" + side] - n_want) <= ties, side
        assert_close(w_l.data, st.w_lhs, rtol, "w_lhs")
        opt_l = trainer.partitioned_optimizers[("l", 0)]
        assert_close(opt_l.state[w_l]["sum"], st.g_lhs, rtol, "g_lhs")
        if not st.shared:
            assert_close(w_r.data, st.w_rhs, rtol, "w_rhs")
        if cfg.global_emb:
            g_l = model.global_embs[pbg.model.MultiRelationEmbedder.EMB_PREFIX + "l"]
            assert_close(g_l.data, st.glob_lhs, rtol, "glob_lhs")
            assert_close(trainer.model_optimizer.state[g_l]["sum"], st.glob_lhs_sum, rtol, "glob_lhs.sum")
            if not st.shared:
                g_r = model.global_embs[pbg.model.MultiRelationEmbedder.EMB_PREFIX + "r"]
                assert_close(g_r.data, st.glob_rhs, rtol, "glob_rhs")
        if not cfg.dynamic and st.rhs_op:
            op = model.rhs_operators[rel]
            for k, v in st.rhs_op.items():
                assert_close(getattr(op, k).data, v[rel], rtol, k)
                assert_close(trainer.model_optimizer.state[getattr(op, k)]["sum"], st.rhs_op_sum[k][rel], rtol, k + ".sum")


def test_model_and_trainer_raise_on_ids_outside_the_table(pbg):
    """An entity id outside its table raises IndexError from MultiRelationEmbedder.forward and from
    Trainer.process_one_batch, as F.embedding does in the reference (model.py:57-61), and leaves the
    table as it was; with Trainer.check_ids switched off the kernels clamp the id instead."""
    say("ids outside the table")
    from tests.test_gpu_step import make_inputs

    cfg = ostep.StepConfig(dim=12, operator="none", comparator="dot", loss="ranking", num_batch_negs=5, num_uniform_negs=4,
                           num_relations=1, relation_weights=[1.0], margin=0.1)
    st, batches = make_inputs(cfg, 20, 50, 1, seed=2)
    model, w_l, _ = build_model(pbg, cfg, st, 1)
    EL, ED, T = pbg.entitylist.EntityList, pbg.edgelist.EdgeList, pbg.train
    loss_fn = pbg.losses.LOSS_FUNCTIONS.get_class(cfg.loss)(margin=cfg.margin)
    trainer = T.Trainer(T.make_optimizer(list(model.parameters()), False, 0.1, 0.1), loss_fn, [1.0])
    trainer.partitioned_optimizers[("l", 0)] = T.make_optimizer([w_l], True, 0.1)
    lhs, rhs, rel, ul, ur = batches[0]
    before = w_l.detach().clone()
    for bad in (50, -1):
        wrong = lhs.clone()
        wrong[3] = bad
        edges = ED(EL.from_tensor(wrong.to(DEV)), EL.from_tensor(rhs.to(DEV)), torch.tensor(rel))
        with pytest.raises(IndexError):
            model(edges, uniform_negs=(ul.to(DEV), ur.to(DEV)))
        trainer.next_uniform_negs = (ul.to(DEV), ur.to(DEV))
        with pytest.raises(IndexError):
            trainer.process_one_batch(model, edges)
        assert torch.equal(before, w_l.detach())
    trainer.check_ids = False
    trainer.next_uniform_negs = (ul.to(DEV), ur.to(DEV))
    trainer.process_one_batch(model, edges)  # the id is clamped to the table's first row
    assert not torch.equal(before, w_l.detach())


def test_row_adagrad_and_async_adagrad_optimizers(pbg):
    torch.manual_seed(0)
    w0 = torch.randn(50, 12)
    p = torch.nn.Parameter(w0.clone().to(DEV))
    opt = pbg.row_adagrad.RowAdagrad([p], lr=0.05)
    ref_w, ref_g = w0.clone(), torch.zeros(50)
    emb = pbg.model.SimpleEmbedding(p)
    for it in range(3):
        idx = torch.randint(0, 50, (40,))
        opt.zero_grad()
        out = emb.get(idx.to(DEV))
        coef = torch.randn(40, 12)
        (out * coef.to(DEV)).sum().backward()
        opt.step()
        ostep.row_adagrad_sparse(ref_w, ref_g, torch.sparse_coo_tensor(idx.unsqueeze(0), coef, (50, 12)), 0.05)
    assert torch.allclose(p.data.cpu(), ref_w, rtol=1e-5, atol=1e-6)
    assert torch.allclose(opt.state[p]["sum"].cpu(), ref_g, rtol=1e-5, atol=1e-7)
    # dense gradient
    p.grad = torch.randn(50, 12, device=DEV)
    dense = p.grad.cpu().clone()
    opt.step()
    ostep.row_adagrad_dense(ref_w, ref_g, dense, 0.05)
    assert torch.allclose(p.data.cpu(), ref_w, rtol=1e-5, atol=1e-6)
    with pytest.raises(RuntimeError, match="weight_decay"):
        o2 = pbg.row_adagrad.RowAdagrad([p], lr=0.05, weight_decay=0.1)
        p.grad = torch.sparse_coo_tensor(torch.tensor([[1]], device=DEV), torch.ones(1, 12, device=DEV), (50, 12))
        o2.step()
    # AsyncAdagrad == torch.optim.Adagrad in one process (test/test_optimizers.py:110-130)
    q0 = torch.randn(7, 5)
    q = torch.nn.Parameter(q0.clone().to(DEV))
    gold = torch.nn.Parameter(q0.clone())
    a, b = pbg.async_adagrad.AsyncAdagrad([q]), torch.optim.Adagrad([gold])
    for _ in range(5):
        g = torch.randn(7, 5)
        q.grad, gold.grad = g.to(DEV), g.clone()
        a.step()
        b.step()
    assert torch.allclose(q.data.cpu(), gold.data, rtol=5e-5, atol=5e-5)


def test_C_module_matches_the_reference_contract(pbg):
    C = pbg._C
    n = 5000
    p = np.random.default_rng(1).permutation(n).astype(np.int64)
    tp = torch.from_numpy(p).to(DEV)
    assert np.array_equal(C.reverse_permutation(tp, 4).cpu().numpy(), operm.reverse_permutation(p))
    t = torch.randn(n, 20)
    td = t.to(DEV)
    assert C.shuffle(td, tp, 4) is None
    assert np.array_equal(td.cpu().numpy(), operm.shuffle(t.numpy(), p))
    with pytest.raises(ValueError, match="out-of-bound"):
        C.shuffle(td, torch.full((n,), n, dtype=torch.int64, device=DEV), 1)
    perm = C.randperm(n, 8, 3)
    assert perm.is_cuda and operm.is_permutation(perm.cpu().numpy())
    assert torch.equal(perm, C.randperm(n, 2, 3))
    assert operm.is_permutation(C.randperm(n, 4).cpu().numpy())
    rng = np.random.default_rng(2)
    lhs = rng.integers(0, 100, n).astype(np.int64)
    rhs = rng.integers(0, 60, n).astype(np.int64)
    rel = rng.integers(0, 2, n).astype(np.int64)
    pl = [rng.permutation(100).astype(np.int64)] * 2
    pr = [rng.permutation(60).astype(np.int64)] * 2
    d = lambda x: torch.from_numpy(x).to(DEV)
    outs = [torch.empty(n, dtype=torch.int64, device=DEV) for _ in range(3)]
    res = C.sub_bucket(d(lhs), d(rhs), d(rel), [100, 100], [d(x) for x in pl], [60, 60], [d(x) for x in pr],
                       outs[0], outs[1], outs[2], 3, 2, 8, False)
    lo, ro, relo, ranges = operm.sub_bucket(lhs, rhs, rel, [100, 100], pl, [60, 60], pr, 3, 2, False)
    assert set(res) == set(ranges)
    for key, (a, b) in ranges.items():
        got = res[key]
        assert np.array_equal(got[0].cpu().numpy(), lo[a:b])
        assert np.array_equal(got[1].cpu().numpy(), ro[a:b])
        assert np.array_equal(got[2].cpu().numpy(), relo[a:b])
        assert got[0].data_ptr() == outs[0][a:b].data_ptr()  # views of the caller's storage


def test_ranking_evaluator(pbg):
    """RankingEvaluator (eval.py:43-86) on batch negatives only (nothing sampled):
    loss, mean rank, MRR and hits@k equal the same formulas on the oracle's scores."""
    say("ranking evaluator")
    from tests.test_gpu_step import make_inputs

    cfg = ostep.StepConfig(dim=16, operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=20,
                           num_uniform_negs=0, num_relations=2, relation_weights=[1.0, 0.5])
    num_pos = 57
    st, batches = make_inputs(cfg, num_pos, 300, 1, seed=9)
    model, w_l, w_r = build_model(pbg, cfg, st, 2)
    EL, ED = pbg.entitylist.EntityList, pbg.edgelist.EdgeList
    loss_fn = pbg.losses.LOSS_FUNCTIONS.get_class(cfg.loss)(margin=cfg.margin)
    evaluator = pbg.eval.RankingEvaluator(loss_fn, list(cfg.relation_weights))
    lhs, rhs, rel, ul, ur = batches[0]
    before = w_l.detach().clone()
    stats = evaluator.process_one_batch(model, ED(EL.from_tensor(lhs.to(DEV)), EL.from_tensor(rhs.to(DEV)), torch.tensor(rel)))
    assert torch.equal(before, w_l.detach())  # evaluation does not train
    want, _ = ostep.forward_backward(cfg, st, lhs, rhs, rel, None, None, keep_scores=True)
    sc = want.scores
    ranks = [(neg >= pos.unsqueeze(1)).sum(1) + 1 for pos, neg in ((sc.lhs_pos, sc.lhs_neg), (sc.rhs_pos, sc.rhs_neg))]
    mean2 = lambda a, b: (float(a.sum()) + float(b.sum())) / 2
    m = stats.metrics
    assert stats.count == num_pos
    assert m["loss"] == pytest.approx(want.loss, rel=1e-5)
    assert m["pos_rank"] == pytest.approx(mean2(*ranks), abs=1.0)  # a score tie may move one rank
    assert m["mrr"] == pytest.approx(mean2(*(r.float().reciprocal() for r in ranks)), abs=0.5)
    for k in (1, 10, 50):
        assert m[f"r{k}"] == pytest.approx(mean2(*(r.le(k) for r in ranks)), abs=1.0)
    assert 0.0 <= m["auc"] <= num_pos
    avg = pbg.stats.Stats.sum([stats]).average()
    assert 0.0 <= avg.metrics["auc"] <= 1.0 and 1.0 <= avg.metrics["pos_rank"] <= 21.0

    # An evaluator that overrides the score hook (a filtered evaluator, eval.py:82-86) needs the score
    # matrices and takes the other way through the same numbers: everything but the sampled AUC is equal.
    class Hooked(pbg.eval.RankingEvaluator):
        seen = 0

        def _adjust_scores(self, scores, batch_edges):
            Hooked.seen += 1
            assert scores.lhs_neg.shape == (num_pos, 20)

    hooked = Hooked(loss_fn, list(cfg.relation_weights)).process_one_batch(
        model, ED(EL.from_tensor(lhs.to(DEV)), EL.from_tensor(rhs.to(DEV)), torch.tensor(rel)))
    assert Hooked.seen == 1
    for key in ("pos_rank", "mrr", "r1", "r10", "r50"):
        assert hooked.metrics[key] == m[key], key
    assert hooked.metrics["loss"] == pytest.approx(m["loss"], rel=1e-5)
    assert abs(hooked.metrics["auc"] - m["auc"]) < 0.35 * num_pos  # two random samples of num_pos pairs each

"""config.half_precision (model.py:504-505,827-829) through the C ABI: the product on
the fp16 matrix instructions against torch's Half bmm, and the step against the
oracle's restatement on Half tensors.  Tolerances are float16's: a score is one
rounding of an fp32 sum (the order of that sum may move it by one unit in the last
place), a gradient row two or three."""
import itertools

import pytest
import torch

from oracle import step as ostep
from tests.test_gpu_step import DEV, make_inputs, pack, say, to_runner

pytestmark = pytest.mark.gpu

EPS16 = 2.0 ** -10  # one unit in the last place of a float16 number, relative


def half_numbers(shape, gen, scale=1.0):
    return (torch.randn(shape, generator=gen) * scale).half().float()


GEMM_SHAPES = [
    # (batch, m, n, k, a_kmajor, b_kmajor): the 64 x 64 tiles, the direct-to-LDS 128 x 128 tiles, their edges
    (3, 50, 100, 100, 0, 0), (2, 50, 100, 1024, 0, 0), (2, 300, 260, 128, 0, 0), (1, 1000, 1100, 256, 0, 0),
    (2, 100, 256, 52, 1, 1), (2, 200, 256, 1000, 1, 1), (2, 52, 256, 100, 0, 1), (1, 300, 512, 1100, 0, 1),
    (2, 7, 5, 3, 0, 0), (1, 130, 131, 18, 0, 0), (1, 132, 136, 36, 1, 0),
]


@pytest.mark.parametrize("batch,m,n,k,akm,bkm", GEMM_SHAPES)
def test_half_product_matches_torch_half_bmm(pbg, batch, m, n, k, akm, bkm):
    say("gemm_f16", batch, m, n, k, akm, bkm)
    g = torch.Generator().manual_seed(m * 1000 + n + k)
    a = half_numbers((batch, k, m) if akm else (batch, m, k), g)
    b = half_numbers((batch, k, n) if bkm else (batch, n, k), g)
    c = torch.full((batch, m, n), float("nan"), device=DEV)
    ad, bd = a.to(DEV), b.to(DEV)
    pbg.native.gemm(ad, bd, c, batch, m, n, k, m if akm else k, n if bkm else k, n, a[0].numel(), b[0].numel(), m * n,
                    akm, bkm, half=True)
    am = a.transpose(1, 2) if akm else a
    bm = b if bkm else b.transpose(1, 2)
    want = torch.bmm(am.half(), bm.half()).float()
    exact = torch.bmm(am.double(), bm.double())
    got = c.cpu()
    assert torch.equal(got.half().float(), got), "the result is made of float16 numbers"
    # within one unit in the last place of the exact product (plus what an fp32 sum of k terms can be off
    # by, which is all that is left of a sum that cancels), and mostly equal to torch's own
    noise = 2.0 ** -23 * torch.bmm(am.double().abs(), bm.double().abs())
    ulp = torch.pow(2.0, torch.floor(torch.log2(exact.abs().clamp_min(2.0 ** -14))) - 10)
    assert bool(((got.double() - exact).abs() <= ulp + noise).all())
    assert float((got != want).float().mean()) < 0.02
    # accumulation onto C (beta = 1), as the backward product of rows that are positives and negatives at once does
    c2 = half_numbers((batch, m, n), g).to(DEV)
    base = c2.cpu().clone()
    pbg.native.gemm(ad, bd, c2, batch, m, n, k, m if akm else k, n if bkm else k, n, a[0].numel(), b[0].numel(), m * n,
                    akm, bkm, beta=1.0, half=True)
    # Two roundings, as autograd adds two Half gradients: the product is a Half tensor of its own, then the sum is
    # rounded -- within a unit of the product plus a unit of the sum of the exact value, and mostly equal to the
    # same two steps on torch's Half tensors.
    want2 = (exact + base.double())
    ulp2 = torch.pow(2.0, torch.floor(torch.log2(want2.abs().clamp_min(2.0 ** -14))) - 10)
    assert bool(((c2.cpu().double() - want2).abs() <= ulp + ulp2 + noise).all())
    twice = (want.half() + base.half()).float()
    assert float((c2.cpu() != twice).float().mean()) < 0.02


HALF_CASES = []
for op, cmp_, loss, dyn in itertools.product(("none", "diagonal", "translation", "complex_diagonal", "linear", "affine"),
                                             ("dot", "cos"), ostep.LOSS_NAMES, (False, True)):
    HALF_CASES.append(dict(operator=op, comparator=cmp_, loss=loss, dynamic=dyn, num_batch_negs=4, num_uniform_negs=3,
                           num_pos=10, dim=6))
HALF_CASES += [
    # the shapes of the BASELINE configurations, reduced: fused and streaming shapes run staged here
    dict(operator="none", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50,
         num_pos=130, dim=100),
    dict(operator="none", comparator="cos", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50,
         num_pos=130, dim=1024),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=50,
         num_uniform_negs=300, num_pos=120, dim=400),
    dict(operator="none", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=200, num_uniform_negs=20,
         num_pos=300, dim=1024),
    dict(operator="linear", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=100,
         num_uniform_negs=100, num_pos=300, dim=256),
    dict(operator="diagonal", comparator="cos", loss="softmax", dynamic=False, num_batch_negs=0, num_uniform_negs=7,
         num_pos=30, dim=9),
    dict(operator="translation", comparator="dot", loss="logistic", dynamic=False, num_batch_negs=4,
         num_uniform_negs=3, num_pos=9, dim=8, disable_lhs_negs=True),
]
# the fused route's shapes (dims that are multiples of 4, batch + uniform negatives on both sides): full and partial
# chunks, dims with and without a remainder of the 16-wide k groups, every tile count
for op, cmp_, loss in itertools.product(("none", "diagonal", "translation"), ("dot", "cos"), ostep.LOSS_NAMES):
    HALF_CASES.append(dict(operator=op, comparator=cmp_, loss=loss, dynamic=False, num_batch_negs=50, num_uniform_negs=50,
                           num_pos=130, dim=100))
HALF_CASES += [
    dict(operator="none", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=64, num_uniform_negs=64, num_pos=200, dim=128),
    dict(operator="none", comparator="cos", loss="softmax", dynamic=False, num_batch_negs=37, num_uniform_negs=20, num_pos=100, dim=64),
    dict(operator="translation", comparator="dot", loss="logistic", dynamic=False, num_batch_negs=16, num_uniform_negs=9, num_pos=40, dim=20),
    dict(operator="diagonal", comparator="cos", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=3, num_pos=75, dim=36),
    dict(operator="none", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=13, num_uniform_negs=64, num_pos=30, dim=112),
]
# rows wider than 128 floats: the chunk kernel on slices (cos: after a pass of its own for the norms)
for op, cmp_, loss in itertools.product(("none", "translation", "diagonal"), ("dot", "cos"), ("ranking", "softmax")):
    HALF_CASES.append(dict(operator=op, comparator=cmp_, loss=loss, dynamic=False, num_batch_negs=50, num_uniform_negs=50,
                           num_pos=130, dim=256))
HALF_CASES += [
    dict(operator="none", comparator="cos", loss="logistic", dynamic=False, num_batch_negs=33, num_uniform_negs=17, num_pos=70, dim=200),
    dict(operator="none", comparator="dot", loss="logistic", dynamic=False, num_batch_negs=16, num_uniform_negs=49, num_pos=40, dim=132),
    # complex_diagonal on slices of 64 coordinate pairs
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=400),
    dict(operator="complex_diagonal", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50, num_pos=100, dim=256),
    dict(operator="complex_diagonal", comparator="dot", loss="logistic", dynamic=False, num_batch_negs=33, num_uniform_negs=17, num_pos=70, dim=136),
]


def close16(got, want, what, units=2.0, floor=None):
    """|got - want| <= units * 2^-10 * max(|want|, floor); floor defaults to a hundredth of the largest |want|"""
    got, want = got.detach().cpu().double(), want.detach().double()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if want.numel() == 0:
        return
    floor = 0.01 * float(want.abs().max()) if floor is None else floor
    bad = (got - want).abs() > units * EPS16 * want.abs().clamp_min(max(floor, 1e-30))
    worst = int(((got - want).abs() / want.abs().clamp_min(max(floor, 1e-30))).argmax())
    assert not bool(bad.any()), (
        f"{what}: max err {float((got - want).abs().max()):.3e}, scale {float(want.abs().max()):.3e}, {int(bad.sum())} of "
        f"{want.numel()} beyond the bound; worst: got {float(got.flatten()[worst])!r}, want {float(want.flatten()[worst])!r}")


@pytest.mark.parametrize("case", HALF_CASES, ids=lambda c: "-".join(str(v) for v in c.values()))
@pytest.mark.parametrize("workers", [1, 3])
def test_half_precision_step(pbg, case, workers):
    say("half", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, half_precision=True, **case)
    n_ent = max(200, num_pos * 4)
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos + dim, shared=(dim % 2 == 0))
    before = [t.clone() for t in (st.w_lhs, st.w_rhs)]
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    assert runner.route in ("staged", "fused")  # (the streaming route does not take half_precision)
    fwd = runner.forward(*pack(cfg, batches))
    torch.cuda.synchronize()
    for k, b in enumerate(batches):
        sc = ostep.forward_backward(cfg, st, *b, keep_scores=True)[0].scores
        got = tuple(t[k].cpu() for t in fwd)
        # Positive scores are fp32 sums over float16 rows (model.py:177), not float16 numbers: on average they agree
        # far better than float16's 2^-12 (a score rounded to float16 would be off by a quarter unit on average).
        # The largest difference may reach a unit: a coordinate that the two fp32 evaluations of prepare() put on
        # different sides of a float16 rounding boundary moves its row's score.
        pos_scale = float(sc.lhs_pos.abs().max())
        pos_diff = (got[0] - sc.lhs_pos).abs()
        assert float(pos_diff.mean()) <= 2e-5 * pos_scale + 1e-7, ("positive scores, mean", float(pos_diff.mean()))
        assert float(pos_diff.max()) <= EPS16 * pos_scale + 1e-7, ("positive scores, max", float(pos_diff.max()))
        for g, w, name in ((got[2], sc.lhs_neg, "lhs_neg"), (got[3], sc.rhs_neg, "rhs_neg")):
            masked = w == -1e9
            assert torch.equal(g == -1e9, masked), name
            assert torch.equal(g[~masked].half().float(), g[~masked]), name + " holds float16 numbers"
            # (a score that cancels to nearly nothing keeps the absolute error of its float16 inputs: the floor)
            if w.numel():
                close16(g[~masked], w[~masked], name, units=3.0, floor=0.05 * float(w[~masked].abs().max()))
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs = ostep.train_lockstep(cfg, st, batches)
    for k, out in enumerate(outs):
        assert float(runner.loss_out[k]) == pytest.approx(out.loss, rel=4 * EPS16, abs=1e-5), ("loss", k)
    # The tables' movement: a row's step is lr * g / sqrt(sum of squares) with g a float16 gradient row, itself
    # a float16 sum of float16 terms: every entry is off by a rounding of the row's larger partial sums, so the
    # bound is two units of the LARGEST step, for every entry.
    for got, want, was, name in ((runner.w_lhs, st.w_lhs, before[0], "w_lhs"), (runner.w_rhs, st.w_rhs, before[1], "w_rhs")):
        step = want - was
        # (cos: prepare's backward takes the row's own direction out of the float16 gradient; what is left is
        # smaller than the gradient whose rounding noise it keeps)
        close16(got.cpu() - was, step, "step of " + name, units=8.0 if cfg.comparator == "cos" else 2.0,
                floor=float(step.abs().max()))
    close16(runner.g_lhs, st.g_lhs, "g_lhs", units=8.0)
    # Operator parameters: AsyncAdagrad's first steps are lr * g / |g|, so an entry whose gradient is float16
    # rounding noise around zero moves by a full step in either direction; a handful of such entries per matrix
    # are held to "within the steps the call can take" instead.
    for name, got, want in (("rhs_op", runner.rhs_op, st.rhs_op), ("lhs_op", runner.lhs_op, st.lhs_op)):
        for k in want:
            g, w = got[k].cpu().double(), want[k].double()
            bound = 4.0 * EPS16 * float(w.abs().max())
            off = (g - w).abs() > bound
            assert int(off.sum()) <= max(2, w.numel() // 20000), (name, k, int(off.sum()), w.numel())
            assert float((g - w).abs().max()) <= 2 * cfg.relation_lr * workers + bound, (name, k)


def test_half_precision_is_refused_where_it_is_not_built(pbg):
    for kw in (dict(comparator="l2"), dict(comparator="squared_l2"), dict(bias=True), dict(regularization_coef=1e-3, operator="diagonal")):
        cfg = ostep.StepConfig(dim=8, num_batch_negs=4, num_uniform_negs=3, half_precision=True, **kw)
        st, _ = make_inputs(cfg, 10, 50, 1, seed=1)
        with pytest.raises(NotImplementedError, match="half_precision"):
            to_runner(pbg, cfg, st, 10, 1)


@pytest.mark.parametrize("case", [
    dict(operator="translation", comparator="cos", loss="softmax", dynamic=False, num_batch_negs=10, num_uniform_negs=10),
    dict(operator="diagonal", comparator="dot", loss="logistic", dynamic=True, num_batch_negs=8, num_uniform_negs=5),
], ids=lambda c: "-".join(str(v) for v in c.values()))
def test_half_precision_through_the_model_classes(pbg, case):
    """MultiRelationEmbedder(half_precision=True) (model.py:409,444) hands the switch to forward and to the
    Trainer's step."""
    say("half model", case)
    from tests.test_gpu_plugins import build_model

    cfg = ostep.StepConfig(dim=16, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01, margin=0.1,
                           half_precision=True, **case)
    st, batches = make_inputs(cfg, 33, 300, 1, seed=5, shared=True)
    model, w_l, w_r = build_model(pbg, cfg, st, 1 if cfg.dynamic else 3)
    assert model.half_precision
    EL, ED, T = pbg.entitylist.EntityList, pbg.edgelist.EdgeList, pbg.train
    lhs, rhs, rel, ul, ur = batches[0]
    rel_t = rel.to(DEV) if cfg.dynamic else torch.tensor(rel)
    edges = ED(EL.from_tensor(lhs.to(DEV)), EL.from_tensor(rhs.to(DEV)), rel_t)
    scores, _ = model(edges, uniform_negs=(ul.to(DEV), ur.to(DEV)))
    want, _ = ostep.forward_backward(cfg, st, lhs, rhs, rel, ul, ur, keep_scores=True)
    got = scores.lhs_neg.cpu()
    masked = want.scores.lhs_neg == -1e9
    assert torch.equal(got == -1e9, masked)
    assert torch.equal(got[~masked].half().float(), got[~masked]), "float16 numbers: the switch reached the kernels"
    close16(got[~masked], want.scores.lhs_neg[~masked], "lhs_neg", units=3.0, floor=0.05 * float(want.scores.lhs_neg[~masked].abs().max()))
    loss_fn = pbg.losses.LOSS_FUNCTIONS.get_class(cfg.loss)(margin=cfg.margin)
    trainer = T.Trainer(T.make_optimizer(list(model.parameters()), False, cfg.lr, cfg.relation_lr), loss_fn, list(cfg.relation_weights))
    trainer.partitioned_optimizers[("l", 0)] = T.make_optimizer([w_l], True, cfg.lr)
    trainer.next_uniform_negs = (ul.to(DEV), ur.to(DEV))
    before = st.w_lhs.clone()
    stats = trainer.process_one_batch(model, edges)
    out = ostep.train_step(cfg, st, lhs, rhs, rel, ul, ur)
    assert float(stats.metrics["loss"]) == pytest.approx(out.loss, rel=4 * EPS16, abs=1e-5)
    step = st.w_lhs - before
    close16(w_l.detach().cpu() - before, step, "step of the table", units=8.0 if cfg.comparator == "cos" else 2.0,
            floor=float(step.abs().max()))

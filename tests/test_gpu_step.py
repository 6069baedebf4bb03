"""GPU parity of the training step through the C ABI against the CPU oracle:
scores / loss / updated tables, Adagrad state and operator parameters within
1e-5 relative after one step, 1e-4 after many; violator counts exact."""
import itertools

import pytest
import torch

from oracle import step as ostep
from tests.parity import anchored_state, double_state, violator_ties

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def say(*a):
    print(*a, flush=True)


def make_inputs(cfg, num_pos, n_ent, workers, seed, shared=True, scale=0.3):
    g = torch.Generator().manual_seed(seed)
    w_l = torch.randn(n_ent, cfg.dim, generator=g) * scale
    w_r = None if shared else torch.randn(n_ent + 5, cfg.dim, generator=g) * scale
    n_r = n_ent if shared else n_ent + 5
    _, c, _ = cfg.chunking(num_pos)
    u = cfg.num_uniform_negs
    batches = []
    for _ in range(workers):
        lhs = torch.randint(0, n_ent, (num_pos,), generator=g)
        rhs = torch.randint(0, n_r, (num_pos,), generator=g)
        ul = torch.randint(0, n_ent, (c, u), generator=g)
        ur = torch.randint(0, n_r, (c, u), generator=g)
        if cfg.dynamic:
            rel = torch.randint(0, cfg.num_relations, (num_pos,), generator=g)
        else:
            rel = int(torch.randint(0, cfg.num_relations, (1,), generator=g))
        batches.append((lhs, rhs, rel, ul, ur))
    st = ostep.make_state(cfg, w_l, w_r)
    for d in (st.lhs_op, st.rhs_op):
        for k in d:
            d[k] = d[k] + 0.2 * torch.randn(d[k].shape, generator=g)
    if st.glob_lhs is not None:
        st.glob_lhs += 0.3 * scale * torch.randn(cfg.dim, generator=g)
        if st.glob_rhs is not st.glob_lhs:
            st.glob_rhs += 0.3 * scale * torch.randn(cfg.dim, generator=g)
    return st, batches


def to_runner(pbg, cfg, st, num_pos, workers):
    spec = pbg.StepSpec(
        dim=cfg.dim, batch_size=num_pos, num_workers=workers, num_batch_negs=cfg.num_batch_negs,
        num_uniform_negs=cfg.num_uniform_negs, disable_lhs_negs=cfg.disable_lhs_negs,
        disable_rhs_negs=cfg.disable_rhs_negs, operator=cfg.operator, dynamic=cfg.dynamic,
        num_relations=cfg.num_relations, comparator=cfg.comparator, loss=cfg.loss, margin=cfg.margin, lr=cfg.lr,
        relation_lr=cfg.relation_lr, regularization_coef=cfg.regularization_coef, max_norm=cfg.max_norm, bias=cfg.bias, all_negs=cfg.all_negs,
        half_precision=cfg.half_precision)
    dev = lambda t: t.clone().to(DEV)
    w_l, g_l = dev(st.w_lhs), dev(st.g_lhs)
    w_r, g_r = (None, None) if st.shared else (dev(st.w_rhs), dev(st.g_rhs))
    ops = [{k: dev(v) for k, v in d.items()} for d in (st.rhs_op, st.rhs_op_sum, st.lhs_op, st.lhs_op_sum)]
    rw = torch.tensor(list(cfg.relation_weights), dtype=torch.float32, device=DEV)
    glob = sums = None
    if st.glob_lhs is not None:
        gl, sl = dev(st.glob_lhs), dev(st.glob_lhs_sum)
        one = st.glob_rhs is st.glob_lhs
        glob, sums = (gl, gl if one else dev(st.glob_rhs)), (sl, sl if one else dev(st.glob_rhs_sum))
    runner = pbg.StepRunner(spec, w_l, g_l, w_r, g_r, ops[0], ops[1], ops[2], ops[3], relation_weights=rw,
                            global_embs=glob, global_sums=sums)
    return runner


def pack(cfg, batches):
    lhs = torch.stack([b[0] for b in batches]).to(DEV)
    rhs = torch.stack([b[1] for b in batches]).to(DEV)
    if cfg.dynamic:
        rel = torch.stack([b[2] for b in batches]).to(DEV)
    else:
        rel = torch.tensor([b[2] for b in batches], dtype=torch.int64, device=DEV)
    ul = torch.stack([b[3] for b in batches]).contiguous().to(DEV)
    ur = torch.stack([b[4] for b in batches]).contiguous().to(DEV)
    return lhs, rhs, rel, ul, ur


def assert_close(got, want, rtol, what, atol_scale=1e-6):
    got = got.detach().cpu().double()
    want = want.detach().double()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if want.numel() == 0:
        return
    scale = want.abs().max().item()
    err = (got - want).abs()
    bound = rtol * want.abs() + atol_scale * max(scale, 1e-30) * rtol / 1e-5
    bad = err > bound
    assert not bad.any(), (what, "max err", err.max().item(), "scale", scale, "count", int(bad.sum()))


def compare_scores(cfg, got, want_scores):
    lp, rp, ln, rn = got
    for name, g, w in (("lhs_pos", lp, want_scores.lhs_pos), ("rhs_pos", rp, want_scores.rhs_pos),
                       ("lhs_neg", ln, want_scores.lhs_neg), ("rhs_neg", rn, want_scores.rhs_neg)):
        g = g.cpu()
        assert g.shape == w.shape, (name, g.shape, w.shape)
        masked = w == -1e9
        assert torch.equal(g == -1e9, masked), name
        if cfg.comparator == "l2":
            # -sqrt(||a||^2 - 2ab + ||b||^2) loses all precision near zero distance
            # (model.py:228-236): compare the squared distances
            assert_close((g * g)[~masked], (w * w)[~masked], 2e-5, name, atol_scale=2e-6)
        else:
            assert_close(g[~masked], w[~masked], 1e-5, name)


FORWARD_CASES = []
for op, cmp_, dyn in itertools.product(ostep.OPERATOR_NAMES, ostep.COMPARATOR_NAMES, (False, True)):
    FORWARD_CASES.append(dict(operator=op, comparator=cmp_, dynamic=dyn, num_batch_negs=4, num_uniform_negs=3,
                              num_pos=10, dim=6))
FORWARD_CASES += [
    dict(operator="none", comparator="dot", dynamic=False, num_batch_negs=50, num_uniform_negs=50, num_pos=1000, dim=100),
    dict(operator="none", comparator="dot", dynamic=False, num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=100),
    dict(operator="complex_diagonal", comparator="dot", dynamic=False, num_batch_negs=50, num_uniform_negs=100,
         num_pos=200, dim=400),
    dict(operator="translation", comparator="l2", dynamic=False, num_batch_negs=50, num_uniform_negs=50, num_pos=173, dim=100),
    dict(operator="linear", comparator="cos", dynamic=False, num_batch_negs=100, num_uniform_negs=100, num_pos=200, dim=256),
    dict(operator="none", comparator="dot", dynamic=False, num_batch_negs=200, num_uniform_negs=20, num_pos=300, dim=1024),
    dict(operator="diagonal", comparator="cos", dynamic=False, num_batch_negs=0, num_uniform_negs=7, num_pos=30, dim=9),
    dict(operator="diagonal", comparator="dot", dynamic=True, num_batch_negs=8, num_uniform_negs=0, num_pos=20, dim=10),
    dict(operator="complex_diagonal", comparator="dot", dynamic=False, num_batch_negs=4, num_uniform_negs=3,
         num_pos=9, dim=8, disable_lhs_negs=True),
    dict(operator="translation", comparator="l2", dynamic=True, num_batch_negs=4, num_uniform_negs=3,
         num_pos=9, dim=8, disable_rhs_negs=True),
    dict(operator="none", comparator="dot", dynamic=False, num_batch_negs=16, num_uniform_negs=2, num_pos=5, dim=7),
    # rows wider than 1024 floats: 32 and 64 floats of a row per lane
    dict(operator="complex_diagonal", comparator="cos", dynamic=False, num_batch_negs=8, num_uniform_negs=5, num_pos=24, dim=2048),
    dict(operator="translation", comparator="l2", dynamic=True, num_batch_negs=8, num_uniform_negs=5, num_pos=24, dim=4096),
    dict(operator="diagonal", comparator="dot", dynamic=False, num_batch_negs=8, num_uniform_negs=5, num_pos=24, dim=2050),
]


def ids(c):
    return "-".join(str(v) for v in c.values())


@pytest.mark.parametrize("case", FORWARD_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_model_forward(pbg, case, workers):
    say("forward", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], **case)
    n_ent = max(50, num_pos * 4)
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos + dim, shared=(dim % 2 == 0))
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    got = runner.forward(*pack(cfg, batches))
    torch.cuda.synchronize()
    for k, b in enumerate(batches):
        _, _ = b[0], b[1]
        out, _ = ostep.forward_backward(cfg, st, *b, keep_scores=True)
        compare_scores(cfg, tuple(t[k] for t in got), out.scores)


TRAIN_CASES = []
for op, cmp_, loss in itertools.product(("none", "diagonal", "translation", "complex_diagonal", "linear"),
                                        ostep.COMPARATOR_NAMES, ostep.LOSS_NAMES):
    TRAIN_CASES.append(dict(operator=op, comparator=cmp_, loss=loss, dynamic=False, num_batch_negs=4,
                            num_uniform_negs=3, num_pos=10, dim=6))
for op, cmp_, loss in itertools.product(ostep.OPERATOR_NAMES, ostep.COMPARATOR_NAMES, ostep.LOSS_NAMES):
    TRAIN_CASES.append(dict(operator=op, comparator=cmp_, loss=loss, dynamic=True, num_batch_negs=4,
                            num_uniform_negs=3, num_pos=10, dim=6))
TRAIN_CASES += [
    dict(operator="none", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50,
         num_pos=1000, dim=100),
    dict(operator="none", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50,
         num_pos=130, dim=100),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=50,
         num_uniform_negs=100, num_pos=200, dim=400),
    dict(operator="translation", comparator="l2", loss="ranking", dynamic=False, num_batch_negs=50,
         num_uniform_negs=50, num_pos=173, dim=100),
    dict(operator="linear", comparator="cos", loss="logistic", dynamic=False, num_batch_negs=100,
         num_uniform_negs=100, num_pos=200, dim=256),
    dict(operator="none", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=200, num_uniform_negs=20,
         num_pos=300, dim=1024),
    dict(operator="diagonal", comparator="cos", loss="softmax", dynamic=False, num_batch_negs=0, num_uniform_negs=7,
         num_pos=30, dim=9),
    dict(operator="complex_diagonal", comparator="dot", loss="logistic", dynamic=False, num_batch_negs=4,
         num_uniform_negs=3, num_pos=9, dim=8, disable_lhs_negs=True),
    dict(operator="translation", comparator="l2", loss="logistic", dynamic=False, num_batch_negs=4,
         num_uniform_negs=3, num_pos=9, dim=8, disable_rhs_negs=True),
    dict(operator="none", comparator="cos", loss="ranking", dynamic=True, num_batch_negs=4, num_uniform_negs=3,
         num_pos=9, dim=8, disable_rhs_negs=True),
    dict(operator="none", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=16, num_uniform_negs=2,
         num_pos=5, dim=7),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=True, num_batch_negs=50,
         num_uniform_negs=100, num_pos=200, dim=400),
    dict(operator="linear", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=100,
         num_uniform_negs=100, num_pos=300, dim=130),
    dict(operator="translation", comparator="l2", loss="ranking", dynamic=True, num_batch_negs=50,
         num_uniform_negs=50, num_pos=173, dim=100),
    dict(operator="diagonal", comparator="dot", loss="logistic", dynamic=True, num_batch_negs=0,
         num_uniform_negs=9, num_pos=40, dim=9, disable_lhs_negs=True),
    # rows wider than 1024 floats (the largest dimension is 4096), also where the dimension is no multiple of 4
    dict(operator="complex_diagonal", comparator="cos", loss="softmax", dynamic=False, num_batch_negs=8,
         num_uniform_negs=5, num_pos=24, dim=2048),
    dict(operator="translation", comparator="l2", loss="ranking", dynamic=True, num_batch_negs=8,
         num_uniform_negs=5, num_pos=24, dim=4096),
    dict(operator="diagonal", comparator="dot", loss="logistic", dynamic=False, num_batch_negs=8,
         num_uniform_negs=5, num_pos=24, dim=1030),
    dict(operator="none", comparator="cos", loss="ranking", dynamic=False, num_batch_negs=8,
         num_uniform_negs=5, num_pos=24, dim=2050),
]


def lockstep(cfg, st, batches, keep_scores=False, anchor=False):
    """oracle.step.train_lockstep on `st`; for the l2 comparator (or with `anchor`) also on a
    float64 copy, the anchor of compare_state's criterion for that comparator."""
    st64 = double_state(st) if cfg.comparator == "l2" or anchor else None
    outs = ostep.train_lockstep(cfg, st, batches, keep_scores=keep_scores)
    if st64 is not None:
        for out, exact in zip(outs, ostep.train_lockstep(cfg, st64, batches)):
            out.exact_loss = exact.loss
    return outs, st64


def loss_close(got, out, rtol=1e-5):
    """The batch's loss within rtol of the CPU path's; with l2, where a zero distance
    evaluates to rounding noise of about 1e-3 (model.py:215-246), alternatively no
    further from the float64 loss than three times the CPU path's fp32 loss is."""
    if got == pytest.approx(out.loss, rel=rtol, abs=1e-6):
        return True
    exact = getattr(out, "exact_loss", None)
    return exact is not None and abs(got - exact) <= rtol * abs(exact) + 1e-6 + 3.0 * abs(out.loss - exact)


def compare_state(cfg, runner, st, rtol, tag, st64=None):
    if st64 is not None:
        # l2 is -sqrt(||a||^2 - 2ab + ||b||^2) (model.py:215-246): near a zero distance the
        # expansion, and through the square root's slope the gradient, is rounding noise in
        # the reference's own fp32 evaluation; there the float64 result is the anchor
        anchored_state(cfg, runner, st, st64, rtol, tag)
        return
    assert_close(runner.w_lhs, st.w_lhs, rtol, tag + " w_lhs")
    assert_close(runner.g_lhs, st.g_lhs, rtol, tag + " g_lhs")
    if not st.shared:
        assert_close(runner.w_rhs, st.w_rhs, rtol, tag + " w_rhs")
        assert_close(runner.g_rhs, st.g_rhs, rtol, tag + " g_rhs")
    for name, got, want in (("rhs_op", runner.rhs_op, st.rhs_op), ("rhs_op_sum", runner.rhs_op_sum, st.rhs_op_sum),
                            ("lhs_op", runner.lhs_op, st.lhs_op), ("lhs_op_sum", runner.lhs_op_sum, st.lhs_op_sum)):
        for k in want:
            assert_close(got[k], want[k], rtol, f"{tag} {name}.{k}")
    if st.glob_lhs is not None:
        assert_close(runner.global_embs[0], st.glob_lhs, rtol, tag + " glob_lhs")
        assert_close(runner.global_sums[0], st.glob_lhs_sum, rtol, tag + " glob_lhs_sum")
        assert_close(runner.global_embs[1], st.glob_rhs, rtol, tag + " glob_rhs")
        assert_close(runner.global_sums[1], st.glob_rhs_sum, rtol, tag + " glob_rhs_sum")


def hinge_ties(cfg, scores, eps=2e-6):
    """Number of negatives whose hinge argument (neg - pos) + margin lies within
    eps of 0 (GPU and CPU scores agree to about 1e-7)."""
    n = 0
    for pos, neg in ((scores.lhs_pos, scores.lhs_neg), (scores.rhs_pos, scores.rhs_neg)):
        x = (neg - pos.unsqueeze(1)) + cfg.margin
        n += int((x.abs() < eps).sum())
    return n


def copy_of(st):
    """An independent copy of an oracle state (one table stays one table)."""
    import copy

    other = copy.deepcopy(st)
    if st.shared:
        other.w_rhs, other.g_rhs = other.w_lhs, other.g_lhs
    if st.glob_lhs is not None and st.glob_rhs is st.glob_lhs:
        other.glob_rhs, other.glob_rhs_sum = other.glob_lhs, other.glob_lhs_sum
    return other


def copy_state(runner, st):
    runner.w_lhs.copy_(st.w_lhs)
    runner.g_lhs.copy_(st.g_lhs)
    if not st.shared:
        runner.w_rhs.copy_(st.w_rhs)
        runner.g_rhs.copy_(st.g_rhs)
    for got, want in ((runner.rhs_op, st.rhs_op), (runner.rhs_op_sum, st.rhs_op_sum),
                      (runner.lhs_op, st.lhs_op), (runner.lhs_op_sum, st.lhs_op_sum)):
        for k in want:
            got[k].copy_(want[k])


@pytest.mark.parametrize("case", TRAIN_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_train_step(pbg, case, workers):
    say("train", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, **case)
    n_ent = max(200, num_pos * 4)
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos + dim, shared=(dim % 2 == 0))
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs, st64 = lockstep(cfg, st, batches, keep_scores=True)
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
        # a negative that IS the positive's entity ties with it up to rounding: the
        # count is exact except for such ties
        sc = out.scores
        for side, pos, neg, want in ((0, sc.lhs_pos, sc.lhs_neg, out.violators_lhs),
                                     (1, sc.rhs_pos, sc.rhs_neg, out.violators_rhs)):
            ties = violator_ties(pos, neg)
            assert abs(int(runner.violators_out[k, side]) - want) <= ties, ("violators", side, k, ties)
    compare_state(cfg, runner, st, rtol, "step", st64)


GLOBAL_CASES = [
    # fused route
    dict(operator="none", comparator="dot", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=200, dim=100),
    # (a distance between two rows of ONE type does not depend on the type's vector: its gradient would be
    # rounding noise, which Adagrad turns into full steps; two types here)
    dict(operator="translation", comparator="l2", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=100,
         shared=False),
    dict(operator="diagonal", comparator="dot", loss="softmax", num_batch_negs=20, num_uniform_negs=10, num_pos=45, dim=32),
    # staged route
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=50, num_uniform_negs=100,
         num_pos=130, dim=400),
    dict(operator="linear", comparator="cos", loss="logistic", num_batch_negs=10, num_uniform_negs=10, num_pos=45, dim=24),
    dict(operator="diagonal", comparator="squared_l2", loss="ranking", num_batch_negs=0, num_uniform_negs=7, num_pos=30,
         dim=9, disable_lhs_negs=True),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=10, num_uniform_negs=5, num_pos=33,
         dim=16, regularization_coef=1e-2),
    dict(operator="none", comparator="cos", loss="logistic", num_batch_negs=10, num_uniform_negs=5, num_pos=33, dim=16,
         shared=False),
]


@pytest.mark.parametrize("case", GLOBAL_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_train_step_with_global_embeddings(pbg, case, workers):
    """config.global_emb (model.py:433-441,486-492): every gathered row is shifted by
    its entity type's vector, which is trained by the model optimizer; one vector
    when the sides share the type (even dim here), two otherwise."""
    say("train+global", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    shared = case.pop("shared", dim % 2 == 0)
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, global_emb=True, **case)
    n_ent = max(200, num_pos * (40 if cfg.comparator == "l2" else 4))
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos + dim, shared=shared)
    zero_glob = (st.glob_lhs.clone(), st.glob_rhs.clone())
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs, st64 = lockstep(cfg, st, batches)
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
    compare_state(cfg, runner, st, rtol, "step+global", st64)
    assert not torch.equal(st.glob_lhs, zero_glob[0])  # it was trained


MAX_NORM_CASES = [
    # fused route, one table and two
    dict(operator="none", comparator="dot", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=200, dim=100),
    dict(operator="translation", comparator="l2", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=100,
         shared=False),
    # staged route
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=50, num_uniform_negs=100,
         num_pos=130, dim=400),
    dict(operator="linear", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=10,
         num_pos=45, dim=24),
    dict(operator="diagonal", comparator="squared_l2", loss="ranking", num_batch_negs=0, num_uniform_negs=7, num_pos=30,
         dim=9, disable_lhs_negs=True, shared=False),
    dict(operator="none", comparator="cos", loss="logistic", num_batch_negs=10, num_uniform_negs=5, num_pos=33, dim=16,
         global_emb=True),
    # cos with a wide negative set: the streaming kernels on the normalised copy of the (renormalised) tables
    dict(operator="none", comparator="cos", loss="softmax", num_batch_negs=50, num_uniform_negs=300, num_pos=130, dim=128),
]


@pytest.mark.parametrize("case", MAX_NORM_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_train_step_with_max_norm(pbg, case, workers):
    """config.max_norm (model.py:61,90-96): rows are looked up with
    F.embedding(max_norm=...), which first scales, IN THE TABLE, every looked-up
    row whose 2-norm exceeds max_norm; about half of the rows here do."""
    say("train+max_norm", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    shared = case.pop("shared", True)
    scale = 0.1
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, max_norm=scale * dim ** 0.5, **case)
    n_ent = max(300, num_pos * (40 if cfg.comparator == "l2" else 6))
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos + dim, shared=shared, scale=scale)
    before = st.w_lhs.clone()
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    # the forward alone renormalises too, as the reference's does
    got = runner.forward(*pack(cfg, batches))
    torch.cuda.synchronize()
    for k, b in enumerate(batches):
        want, _ = ostep.forward_backward(cfg, st, *b, keep_scores=True)
        compare_scores(cfg, tuple(t[k] for t in got), want.scores)
    touched = torch.cat([b[0] for b in batches])
    norms = runner.w_lhs[touched.to(DEV)].norm(dim=1).cpu()
    assert float(norms.max()) <= cfg.max_norm * (1 + 1e-6)
    assert int((before[touched].norm(dim=1) > cfg.max_norm).sum()) > 0  # some rows were too long
    assert_close(runner.w_lhs, st.w_lhs, 1e-6, "renormalised table")
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    # (hundreds of exponentials per score row: the CPU path's own fp32 result is then further from the exact one
    # than the tolerance, and the float64 run anchors the comparison, as in tests/test_gpu_stream.py)
    outs, st64 = lockstep(cfg, st, batches, anchor=runner.route == "stream")
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
    compare_state(cfg, runner, st, rtol, "step+max_norm", st64)


# (A translation moves the bias of every row of its side by the same amount, which ranking and softmax do
# not see: its first element then has a zero gradient, rounding noise that Adagrad would turn into full
# steps -- in the reference too.  Translations are paired with the logistic loss here.)
BIAS_CASES = [
    # shapes the fused kernel would take without the bias
    dict(operator="none", comparator="dot", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=100),
    dict(operator="translation", comparator="squared_l2", loss="logistic", num_batch_negs=20, num_uniform_negs=10, num_pos=45,
         dim=32),
    dict(operator="diagonal", comparator="squared_l2", loss="softmax", num_batch_negs=20, num_uniform_negs=10, num_pos=45,
         dim=32),
    dict(operator="diagonal", comparator="cos", loss="logistic", num_batch_negs=10, num_uniform_negs=5, num_pos=33, dim=16,
         shared=False),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=50, num_uniform_negs=100,
         num_pos=130, dim=400),
    dict(operator="linear", comparator="cos", loss="ranking", num_batch_negs=10, num_uniform_negs=10, num_pos=45, dim=24),
    dict(operator="affine", comparator="dot", loss="logistic", num_batch_negs=8, num_uniform_negs=0, num_pos=30, dim=12),
    dict(operator="diagonal", comparator="squared_l2", loss="ranking", num_batch_negs=0, num_uniform_negs=7, num_pos=30,
         dim=9, disable_lhs_negs=True),
    dict(operator="none", comparator="dot", loss="logistic", num_batch_negs=10, num_uniform_negs=5, num_pos=33, dim=16,
         global_emb=True),  # (a global embedding's first element is such a common shift too)
    # l2: the score matrix holds dLoss/d(squared distance), so dLoss/dscore is kept beside it for the biases' sums
    dict(operator="none", comparator="l2", loss="logistic", num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=100, shared=False),
    dict(operator="diagonal", comparator="l2", loss="ranking", num_batch_negs=20, num_uniform_negs=10, num_pos=45, dim=32),
    dict(operator="complex_diagonal", comparator="l2", loss="softmax", num_batch_negs=10, num_uniform_negs=100, num_pos=33, dim=16,
         shared=False),
    dict(operator="linear", comparator="l2", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=10, num_pos=45,
         dim=24),
    dict(operator="diagonal", comparator="l2", loss="logistic", dynamic=True, num_batch_negs=0, num_uniform_negs=6, num_pos=21,
         dim=10, disable_lhs_negs=True),
    # with the N3 regularizer: the bias is a coordinate of the regularized row (model.py:311-314, regularizers.py:82-97)
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=50, num_uniform_negs=100, num_pos=130,
         dim=400, regularization_coef=1e-3),
    dict(operator="diagonal", comparator="cos", loss="logistic", num_batch_negs=10, num_uniform_negs=5, num_pos=33, dim=16,
         regularization_coef=0.05, shared=False),
    dict(operator="diagonal", comparator="l2", loss="ranking", num_batch_negs=8, num_uniform_negs=4, num_pos=30, dim=10,
         regularization_coef=0.05),
    dict(operator="complex_diagonal", comparator="dot", loss="logistic", dynamic=True, num_batch_negs=20, num_uniform_negs=10,
         num_pos=70, dim=32, regularization_coef=1e-2),
    dict(operator="translation", comparator="squared_l2", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=0,
         num_pos=45, dim=12, regularization_coef=0.02, disable_rhs_negs=True),
    # one relation per edge
    dict(operator="translation", comparator="dot", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=5,
         num_pos=33, dim=16),
    dict(operator="diagonal", comparator="dot", loss="ranking", dynamic=True, num_batch_negs=10, num_uniform_negs=5,
         num_pos=33, dim=16),
    dict(operator="complex_diagonal", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=20, num_uniform_negs=10,
         num_pos=70, dim=32),
    dict(operator="linear", comparator="squared_l2", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=10,
         num_pos=45, dim=24),
    dict(operator="diagonal", comparator="dot", loss="logistic", dynamic=True, num_batch_negs=8, num_uniform_negs=4,
         num_pos=30, dim=9, disable_rhs_negs=True),
    dict(operator="affine", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=0, num_uniform_negs=6,
         num_pos=21, dim=10),
]


@pytest.mark.parametrize("case", BIAS_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_train_step_with_bias(pbg, case, workers):
    """config.bias (BiasedComparator, model.py:306-344): a row's first coordinate
    stays out of the comparator and is added to every score of the row."""
    say("train+bias", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    shared = case.pop("shared", True)
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, bias=True, **case)
    st, batches = make_inputs(cfg, num_pos, max(200, num_pos * 4), workers, seed=num_pos + dim, shared=shared)
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    assert not runner.fused
    got = runner.forward(*pack(cfg, batches))
    for k, b in enumerate(batches):
        want, _ = ostep.forward_backward(cfg, st, *b, keep_scores=True)
        compare_scores(cfg, tuple(t[k] for t in got), want.scores)
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs, st64 = lockstep(cfg, st, batches)
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
        if cfg.regularization_coef:
            assert out.reg > 0.0 and float(runner.reg_out[k]) == pytest.approx(out.reg, rel=1e-5), ("reg", k)
    compare_state(cfg, runner, st, 1e-5, "step+bias", st64)


ALL_NEGS_CASES = [
    dict(operator="none", comparator="dot", loss="softmax", num_pos=64, dim=100),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_pos=130, dim=64, shared=False),
    dict(operator="translation", comparator="l2", loss="ranking", num_pos=45, dim=32),
    dict(operator="diagonal", comparator="cos", loss="logistic", num_pos=33, dim=16, disable_lhs_negs=True, shared=False),
    dict(operator="linear", comparator="squared_l2", loss="ranking", num_pos=30, dim=24),
    dict(operator="diagonal", comparator="dot", loss="logistic", num_pos=40, dim=16, bias=True),
    dict(operator="translation", comparator="dot", loss="softmax", num_pos=33, dim=16, dynamic=True, shared=False),
    dict(operator="linear", comparator="cos", loss="ranking", num_pos=45, dim=24, dynamic=True),
    dict(operator="none", comparator="cos", loss="logistic", num_pos=50, dim=16, global_emb=True, max_norm=1.1),
]


@pytest.mark.parametrize("case", ALL_NEGS_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_train_step_with_all_negs(pbg, case, workers):
    """RelationSchema.all_negs (model.py:648-650,582-618): one chunk, every entity
    of a side's type is a negative, the edge's own entity masked."""
    say("train+all_negs", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    shared = case.pop("shared", True)
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, all_negs=True, num_batch_negs=7, num_uniform_negs=0, **case)
    n_ent = 150 if cfg.comparator != "l2" else 1500
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos + dim, shared=shared)
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    got = runner.forward(*pack(cfg, batches))
    assert got[2].shape[-1] == (0 if cfg.disable_lhs_negs else st.w_lhs.shape[0]) and got[3].shape[-1] == st.w_rhs.shape[0]
    for k, b in enumerate(batches):
        want, _ = ostep.forward_backward(cfg, st, *b, keep_scores=True)
        compare_scores(cfg, tuple(t[k] for t in got), want.scores)
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs, st64 = lockstep(cfg, st, batches)
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
    compare_state(cfg, runner, st, rtol, "step+all_negs", st64)


WEIGHT_CASES = [
    # the single-kernel route (chunk in LDS), each loss
    dict(operator="none", comparator="dot", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=230, dim=100),
    dict(operator="translation", comparator="l2", loss="logistic", num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=100,
         shared=False),
    dict(operator="diagonal", comparator="dot", loss="softmax", num_batch_negs=20, num_uniform_negs=10, num_pos=45, dim=32),
    # the staged route, each loss
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=50, num_uniform_negs=100,
         num_pos=130, dim=400),
    dict(operator="linear", comparator="cos", loss="logistic", num_batch_negs=10, num_uniform_negs=10, num_pos=45, dim=24),
    dict(operator="diagonal", comparator="squared_l2", loss="ranking", num_batch_negs=0, num_uniform_negs=7, num_pos=30,
         dim=9, disable_lhs_negs=True),
    dict(operator="linear", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=10,
         num_pos=45, dim=24),
    dict(operator="translation", comparator="dot", loss="ranking", dynamic=True, num_batch_negs=10, num_uniform_negs=5,
         num_pos=33, dim=16, shared=False),
]


@pytest.mark.parametrize("case", WEIGHT_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_train_step_with_edge_weights(pbg, case, workers):
    """EdgeList.weight (edgelist.py:51-95) inside the step: every loss scales an edge's
    term by its weight (losses.py:65-79, 104-113, 147-161)."""
    say("train+weights", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    shared = case.pop("shared", True)
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, **case)
    n_ent = max(200, num_pos * (40 if cfg.comparator == "l2" else 4))
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos + dim, shared=shared)
    g = torch.Generator().manual_seed(99)
    weights = [0.25 + 2.0 * torch.rand(num_pos, generator=g) for _ in batches]
    weights[0][::7] = 0.0  # (an edge of weight 0 contributes nothing)
    unweighted = copy_of(st)
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    runner.train(*pack(cfg, batches), edge_weight=torch.stack(weights).to(DEV))
    torch.cuda.synchronize()
    outs, st64 = lockstep(cfg, st, [b + (w,) for b, w in zip(batches, weights)])
    ostep.train_lockstep(cfg, unweighted, batches)
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
    compare_state(cfg, runner, st, rtol, "step+weights", st64)
    # the weights moved the result: the comparison above would not pass without them
    assert (st.w_lhs - unweighted.w_lhs).abs().max() > 1e-3 * st.w_lhs.abs().max()
    # what the binding refuses: a host tensor, another dtype, another length
    lhs, rhs, rel, ul, ur = pack(cfg, batches)
    good = torch.stack(weights).to(DEV)
    for bad, err in ((good.cpu(), TypeError), (good.double(), TypeError), (good.flatten()[:-1], ValueError)):
        with pytest.raises(err):
            runner.train(lhs, rhs, rel, ul, ur, edge_weight=bad)


def test_ids_out_of_range_are_found_when_asked(pbg):
    """The kernels clamp ids; StepRunner.train(check_ids=True) raises the IndexError
    the reference's F.embedding raises (model.py:60-61), before anything is trained."""
    say("check_ids")
    cfg = ostep.StepConfig(dim=16, operator="translation", comparator="dot", loss="ranking", num_relations=3,
                           num_batch_negs=5, num_uniform_negs=5, lr=0.1, relation_lr=0.01, margin=0.1)
    st, batches = make_inputs(cfg, 20, 50, 2, seed=5, shared=True)
    runner = to_runner(pbg, cfg, st, 20, 2)
    lhs, rhs, rel, ul, ur = pack(cfg, batches)
    before = runner.w_lhs.clone()
    runner.train(lhs, rhs, rel, ul, ur, check_ids=True)  # in range: trains
    torch.cuda.synchronize()
    assert not torch.equal(before, runner.w_lhs)
    after = runner.w_lhs.clone()
    for which, value in ((0, 50), (1, -1), (2, 3), (3, 50), (4, -7)):
        args = [lhs.clone(), rhs.clone(), rel.clone(), ul.clone(), ur.clone()]
        args[which].view(-1)[-1] = value
        with pytest.raises(IndexError):
            runner.train(*args, check_ids=True)
    torch.cuda.synchronize()
    assert torch.equal(after, runner.w_lhs)


def test_global_embeddings_are_refused_for_dynamic_relations(pbg):
    spec = pbg.StepSpec(dim=8, batch_size=10, dynamic=True, num_relations=2)
    w = torch.randn(20, 8, device=DEV)
    g = torch.zeros(8, device=DEV)
    with pytest.raises(RuntimeError, match="Cannot have global embs with dynamic rels"):
        pbg.StepRunner(spec, w, torch.zeros(20, device=DEV), global_embs=(g, g), global_sums=(g.clone(), g.clone()))


REG_CASES = [
    # the reference's FB15k example: ComplEx, softmax, N3 with coefficient 1e-3 (fb15k_config_cpu.py:33-41)
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=50,
         num_uniform_negs=100, num_pos=130, dim=400, regularization_coef=1e-3),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=True, num_batch_negs=20,
         num_uniform_negs=10, num_pos=70, dim=32, regularization_coef=1e-2),
    dict(operator="diagonal", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=8, num_uniform_negs=4,
         num_pos=30, dim=9, regularization_coef=0.05),
    dict(operator="diagonal", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=8, num_uniform_negs=4,
         num_pos=30, dim=10, regularization_coef=0.05),
    dict(operator="translation", comparator="l2", loss="ranking", dynamic=False, num_batch_negs=10, num_uniform_negs=10,
         num_pos=45, dim=12, regularization_coef=0.02),
    dict(operator="translation", comparator="dot", loss="softmax", dynamic=True, num_batch_negs=10, num_uniform_negs=0,
         num_pos=45, dim=12, regularization_coef=0.02, disable_rhs_negs=True),
    # shapes the fused kernel would take without a regularizer
    dict(operator="none", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50,
         num_pos=200, dim=100, regularization_coef=0.01),
    dict(operator="none", comparator="dot", loss="softmax", dynamic=True, num_batch_negs=6, num_uniform_negs=3,
         num_pos=20, dim=8, regularization_coef=0.1),
]


RANK_CASES = [
    dict(operator="none", comparator="dot", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=230, dim=100),
    dict(operator="none", comparator="cos", loss="softmax", num_batch_negs=20, num_uniform_negs=300, num_pos=90, dim=32),
    dict(operator="translation", comparator="l2", loss="ranking", num_batch_negs=16, num_uniform_negs=40, num_pos=70, dim=24,
         shared=False),
    dict(operator="complex_diagonal", comparator="dot", loss="logistic", dynamic=True, num_batch_negs=10, num_uniform_negs=25,
         num_pos=45, dim=16),
    dict(operator="diagonal", comparator="squared_l2", loss="softmax", num_batch_negs=0, num_uniform_negs=64, num_pos=40, dim=20),
    dict(operator="linear", comparator="cos", loss="logistic", num_batch_negs=12, num_uniform_negs=0, num_pos=30, dim=16,
         disable_lhs_negs=True),
    dict(operator="none", comparator="dot", loss="softmax", num_batch_negs=8, num_uniform_negs=8, num_pos=20, dim=12, bias=True),
    dict(operator="none", comparator="dot", loss="ranking", num_batch_negs=7, num_uniform_negs=0, num_pos=25, dim=12,
         all_negs=True),
]


@pytest.mark.parametrize("case", RANK_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_model_ranks(pbg, case, workers):
    """pbg_model_ranks (the evaluator's ranks, loss and AUC count without the [B, N]
    score matrices, eval.py:57-81) against the matrices of pbg_model_forward -- the
    ranks count `negative >= positive` over the very same floats, so they are equal
    bit for bit -- and against the oracle's loss; the AUC count against the exact
    fraction of (positive, negative) pairs with positive > negative."""
    say("ranks", case, workers)
    case = dict(case)
    num_pos, dim, shared = case.pop("num_pos"), case.pop("dim"), case.pop("shared", True)
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], margin=0.1, **case)
    st, batches = make_inputs(cfg, num_pos, 300, workers, seed=3 * num_pos + dim, shared=shared)
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    args = pack(cfg, batches)
    g = torch.Generator().manual_seed(5)
    weight = (torch.rand(workers, num_pos, generator=g) + 0.5).to(DEV)
    lp, rp, ln, rn = runner.forward(*args)
    samples = 200_000
    for ew in (None, weight):
        glp, grp, lrank, rrank, loss_edge, hits = runner.ranks(*args, edge_weight=ew, auc_samples=samples, auc_seed=11)
        torch.cuda.synchronize()
        assert torch.equal(glp, lp) and torch.equal(grp, rp)
        for side, (pos, neg, rank) in enumerate(((lp, ln, lrank), (rp, rn, rrank))):
            if neg.shape[-1] == 0:
                assert int(rank.abs().sum()) == 0
                continue
            assert torch.equal(rank, (neg >= pos.unsqueeze(-1)).sum(-1) + 1), side
            exact = float((pos.reshape(-1, 1) > neg.reshape(1, -1)).double().mean())
            sigma = (max(exact * (1 - exact), 1e-4) / samples) ** 0.5
            assert abs(int(hits[side]) / samples - exact) < 6 * sigma + 1e-4, (side, int(hits[side]) / samples, exact)
        for k, b in enumerate(batches):
            w = None if ew is None else ew[k].cpu()
            out = ostep.forward_backward(cfg, copy_of(st), *b, weight=w)[0]
            assert float(loss_edge[k].double().sum()) == pytest.approx(out.loss, rel=2e-5, abs=1e-6), (k, ew is not None)


@pytest.mark.parametrize("case", REG_CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_train_step_with_n3_regularizer(pbg, case, workers):
    """(loss + reg).backward() (train_cpu.py:102-103) with the N3 regularizer
    (regularizers.py:51-97): loss, regularizer value, tables, Adagrad sums and
    operator parameters against the oracle."""
    say("train+N3", case, workers)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01,
                           margin=0.1, **case)
    n_ent = max(200, num_pos * (40 if cfg.comparator == "l2" else 4))
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos + dim, shared=(dim % 2 == 0))
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    assert not runner.fused
    before = runner.w_lhs.clone()
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    plain = ostep.StepConfig(**{**cfg.__dict__, "regularization_coef": 0.0})
    st_plain = ostep.TrainState(**{k: (v.clone() if torch.is_tensor(v) else {n: t.clone() for n, t in v.items()})
                                   for k, v in st.__dict__.items() if v is not None})
    if st.shared:
        st_plain.w_rhs, st_plain.g_rhs = st_plain.w_lhs, st_plain.g_lhs
    outs, st64 = lockstep(cfg, st, batches)
    ostep.train_lockstep(plain, st_plain, batches)
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
        assert out.reg > 0.0
        assert float(runner.reg_out[k]) == pytest.approx(out.reg, rel=1e-5), ("reg", k)
    compare_state(cfg, runner, st, rtol, "step+N3", st64)
    # the regularizer moved the result: the comparison above would not pass without it
    assert (st.w_lhs - st_plain.w_lhs).abs().max() > 100 * rtol * (st.w_lhs - before.cpu()).abs().max()


def test_regularizer_is_refused_for_linear(pbg):
    spec = pbg.StepSpec(dim=8, batch_size=10, operator="linear", regularization_coef=1e-3)
    w = torch.randn(20, 8, device=DEV)
    with pytest.raises((RuntimeError, NotImplementedError), match="Regularizer not implemented"):
        pbg.StepRunner(spec, w, torch.zeros(20, device=DEV), rhs_op={"linear_transformation": torch.eye(8, device=DEV)[None]},
                       rhs_op_sum={"linear_transformation": torch.zeros(1, 8, 8, device=DEV)})


@pytest.mark.parametrize("case", [
    dict(operator="none", comparator="dot", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=200, dim=100),
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=20, num_uniform_negs=30, num_pos=100, dim=40),
    dict(operator="translation", comparator="cos", loss="logistic", num_batch_negs=10, num_uniform_negs=10, num_pos=50, dim=16),
    # cfg4's step: translation, l2, ranking, two tables, power-law ids
    dict(operator="translation", comparator="l2", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=200, dim=100,
         shared=False, zipf=1.8),
    # cfg5's step: linear, cos, logistic, one relation per edge
    dict(operator="linear", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=50, num_uniform_negs=50,
         num_pos=100, dim=64),
], ids=ids)
def test_hundred_steps(pbg, case):
    """Updated embeddings, Adagrad state and operator parameters after 100
    sequential steps stay within 1e-4 relative of the CPU path: ONE run of 100
    steps on the GPU and one on the oracle, neither ever seeing the other's state.

    max(0, x) has a gradient of 0 on one side of x = 0 and 1 on the other, so two
    correct fp32 evaluations of a hinge argument within rounding distance of 0 may
    take different sides, and the runs then part for good (every later hinge near
    the changed rows may flip too): on such a batch no tolerance means anything.
    The ranking cases therefore draw their batches along a float64 run of the
    oracle and redraw a batch in which some live hinge argument lies within 4e-6
    of 0, relative to the largest score (the GPU's and the CPU's scores agree to
    about 1e-7); how many were redrawn is printed."""
    from tests.parity import double_state, tie_free_batches, zipf_ids

    say("hundred", case)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    shared, zipf = case.pop("shared", True), case.pop("zipf", None)
    cfg = ostep.StepConfig(dim=dim, num_relations=2, relation_weights=[1.0, 1.0], lr=0.1,
                           dynamic=case.pop("dynamic", False), **case)
    steps = 100
    st, batches = make_inputs(cfg, num_pos, 2000, steps * (5 if cfg.loss == "ranking" else 1), seed=1, shared=shared,
                              scale=1e-3 if case["operator"] == "none" else 0.1)
    if zipf:
        g = torch.Generator().manual_seed(2)
        batches = [(zipf_ids(num_pos, 2000, zipf, g), zipf_ids(num_pos, 2000, zipf, g)) + b[2:] for b in batches]
    st64 = double_state(st)
    if cfg.loss == "ranking":
        batches, drawn = tie_free_batches(cfg, st64, batches, steps, 4e-6)  # (advances st64 through the kept batches)
        say("  batches drawn for", steps, "steps without a hinge tie:", drawn)
    else:
        for b in batches:
            ostep.train_step(cfg, st64, *b)
    assert len(batches) == steps
    runner = to_runner(pbg, cfg, st, num_pos, 1)
    for b in batches:
        runner.train(*pack(cfg, [b]))
        ostep.train_step(cfg, st, *b)
    torch.cuda.synchronize()
    compare_state(cfg, runner, st, 1e-4, "100 steps", st64 if cfg.comparator == "l2" else None)


@pytest.mark.parametrize("workers", [1, 8])
def test_hip_graph_replays_match_eager(pbg, workers):
    """A captured step replayed with new inputs does what the eager call does:
    two runners from the same state, one eager, one replaying its graph, with
    eager work and synchronisations between the replays, stay bit-identical.
    With 8 batches of 1000 edges the call has 160 chunks, enough for the sort of
    its keys to run on the library's side stream beside the chunk kernel: the
    capture then holds a fork and a join."""
    say("hip graph", workers)
    cfg = ostep.StepConfig(dim=100, operator="translation", comparator="l2", loss="ranking", num_batch_negs=50,
                           num_uniform_negs=50, lr=0.1, num_relations=3, relation_weights=[1.0, 0.5, 2.0])
    num_pos, steps = (230, 4) if workers == 1 else (1000, 3)
    st, all_batches = make_inputs(cfg, num_pos, 3000 if workers == 1 else 40000, (steps + 1) * workers, seed=5)
    batches = [all_batches[i * workers:(i + 1) * workers] for i in range(steps + 1)]
    eager = to_runner(pbg, cfg, st, num_pos, workers)
    graphed = to_runner(pbg, cfg, st, num_pos, workers)
    static = [t.clone() for t in pack(cfg, batches[0])]
    graph = graphed.capture_train(*static)  # runs batch 0 twice (set-up call + capture is not a run) ...
    copy_state(graphed, st)                 # ... so start again from the common state
    graphed.loss_out.zero_()
    for b in batches[1:]:
        inputs = pack(cfg, b)
        eager.train(*inputs)
        for dst, src in zip(static, inputs):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        _ = (eager.w_lhs.sum() + graphed.w_lhs.sum()).item()  # unrelated eager work between replays
        assert torch.equal(eager.loss_out, graphed.loss_out)
        assert torch.equal(eager.violators_out, graphed.violators_out)
        assert torch.equal(eager.w_lhs, graphed.w_lhs) and torch.equal(eager.g_lhs, graphed.g_lhs)
        for k in eager.rhs_op:
            assert torch.equal(eager.rhs_op[k], graphed.rhs_op[k])
            assert torch.equal(eager.rhs_op_sum[k], graphed.rhs_op_sum[k])


def test_two_streams_share_the_side_stream(pbg):
    """Two runners train on two streams at once, each call large enough for the sort of
    its keys to run on the library's side stream: the results are those of the same
    calls made one after the other."""
    say("two streams")
    cfg = ostep.StepConfig(dim=100, operator="none", comparator="dot", loss="ranking", num_batch_negs=50,
                           num_uniform_negs=50, lr=0.1)
    workers, num_pos, calls = 8, 1000, 6
    states, inputs = [], []
    for r in range(2):
        st, batches = make_inputs(cfg, num_pos, 50000, workers * calls, seed=11 + r)
        states.append(st)
        inputs.append([pack(cfg, batches[i * workers:(i + 1) * workers]) for i in range(calls)])
    alone = [to_runner(pbg, cfg, st, num_pos, workers) for st in states]
    for r in range(2):
        for inp in inputs[r]:
            alone[r].train(*inp)
    torch.cuda.synchronize()
    together = [to_runner(pbg, cfg, st, num_pos, workers) for st in states]
    streams = [torch.cuda.Stream(device=DEV) for _ in range(2)]
    torch.cuda.synchronize()
    for i in range(calls):
        for r in range(2):
            with torch.cuda.stream(streams[r]):
                together[r].train(*inputs[r][i])
    torch.cuda.synchronize()
    for r in range(2):
        assert together[r].route == "fused"
        assert torch.equal(alone[r].w_lhs, together[r].w_lhs) and torch.equal(alone[r].g_lhs, together[r].g_lhs)
        assert torch.equal(alone[r].loss_out, together[r].loss_out)


@pytest.mark.parametrize("case", [
    dict(operator="none", comparator="dot", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50,
         num_pos=230, dim=100),                                                  # fused chunk kernel
    dict(operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, num_batch_negs=20,
         num_uniform_negs=30, num_pos=70, dim=40),                               # staged kernels, parameter gradient
    dict(operator="translation", comparator="cos", loss="logistic", dynamic=True, num_batch_negs=0,
         num_uniform_negs=9, num_pos=40, dim=10),                                # uniform negatives only
], ids=ids)
def test_negatives_drawn_in_the_step(pbg, case):
    """A step that draws its uniform negatives from a seed is bit-identical to a
    step that is handed pbg_sample_uniform_negatives(seed) and the draw is uniform
    over the table."""
    say("in-step negatives", case)
    from pytorch_biggraph_amd import native

    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    cfg = ostep.StepConfig(dim=dim, num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, **case)
    workers, n_ent, seed = 3, 700, 0x1234567890ABCDEF
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=3, shared=False)
    lhs, rhs, rel, _, _ = pack(cfg, batches)
    a = to_runner(pbg, cfg, st, num_pos, workers)
    b = to_runner(pbg, cfg, st, num_pos, workers)
    shape = (workers, a.spec.num_chunks, cfg.num_uniform_negs)
    ul = native.sample_uniform_negatives(seed, 0, st.w_lhs.shape[0], shape, DEV)
    ur = native.sample_uniform_negatives(seed, 1, st.w_rhs.shape[0], shape, DEV)
    assert int(ul.min()) >= 0 and int(ul.max()) < st.w_lhs.shape[0]
    assert int(ur.min()) >= 0 and int(ur.max()) < st.w_rhs.shape[0]
    assert not torch.equal(ul, ur)
    a.train(lhs, rhs, rel, ul, ur)
    b.train(lhs, rhs, rel, uniform_seed=seed)
    torch.cuda.synchronize()
    assert torch.equal(a.loss_out, b.loss_out) and torch.equal(a.violators_out, b.violators_out)
    for x, y in ((a.w_lhs, b.w_lhs), (a.g_lhs, b.g_lhs), (a.w_rhs, b.w_rhs), (a.g_rhs, b.g_rhs)):
        assert torch.equal(x, y)
    for k in a.rhs_op:
        assert torch.equal(a.rhs_op[k], b.rhs_op[k])
    with pytest.raises(ValueError):
        b.train(lhs, rhs, rel, ul, ur, uniform_seed=seed)
    # uniformity: 200 000 draws over 1000 rows, chi-square with 999 degrees of freedom (mean 999, sd 44.7)
    draws = native.sample_uniform_negatives(seed + 1, 0, 1000, (200_000,), DEV)
    counts = torch.bincount(draws, minlength=1000).double()
    chi2 = float(((counts - 200.0) ** 2 / 200.0).sum())
    assert 999 - 6 * 44.7 < chi2 < 999 + 6 * 44.7, chi2
    other = native.sample_uniform_negatives(seed + 2, 0, 1000, (200_000,), DEV)
    assert float((draws == other).double().mean()) < 0.01


def _fused_shape_cases():
    """A fixed pseudo-random sample of the shapes the LDS-resident chunk kernel
    accepts (and a few just outside, which take the staged kernels)."""
    import random

    rng = random.Random(7)
    cases = []
    for _ in range(48):
        p = rng.choice([1, 2, 3, 15, 16, 17, 31, 33, 48, 50, 63, 64])
        u = rng.choice([1, 2, 5, 16, 17, 49, 50, 64])
        d = rng.choice([4, 8, 12, 36, 60, 64, 100, 116, 124, 128])
        chunks = rng.choice([1, 2, 3])
        num_pos = max(1, p * chunks - rng.choice([0, 0, 1, p // 2]))
        cases.append(dict(operator=rng.choice(["none", "translation", "diagonal"]), comparator=rng.choice(["dot", "l2"]),
                          loss=rng.choice(["ranking", "logistic", "softmax"]), dynamic=False, num_batch_negs=p,
                          num_uniform_negs=u, num_pos=num_pos, dim=d))
    return cases


def _fused_cos_cases():
    """The same kind of sample for the cos comparator (the reference's default,
    config.py:185-190), whose rows are normalised on their way into LDS and whose
    gradient rows go back through the normalisation on their way out."""
    import random

    rng = random.Random(11)
    cases = [dict(operator="none", comparator="cos", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=50,
                  num_pos=173, dim=100)]
    for _ in range(26):
        p = rng.choice([1, 2, 3, 15, 16, 17, 31, 33, 48, 50, 63, 64])
        u = rng.choice([1, 2, 5, 16, 17, 49, 50, 64])
        d = rng.choice([4, 8, 12, 36, 60, 64, 100, 116, 124, 128])
        chunks = rng.choice([1, 2, 3])
        num_pos = max(1, p * chunks - rng.choice([0, 0, 1, p // 2]))
        cases.append(dict(operator=rng.choice(["none", "translation", "diagonal"]), comparator="cos",
                          loss=rng.choice(["ranking", "logistic", "softmax"]), dynamic=False, num_batch_negs=p,
                          num_uniform_negs=u, num_pos=num_pos, dim=d))
    return cases


@pytest.mark.parametrize("case", _fused_shape_cases() + _fused_cos_cases(), ids=ids)
def test_fused_kernel_shapes(pbg, case):
    """Chunk sizes, negative counts, dims and partial last chunks around the
    tile borders of the fused chunk kernel, two batches per call."""
    say("fused shapes", case)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    cfg = ostep.StepConfig(dim=dim, num_relations=2, relation_weights=[1.0, 0.5], lr=0.1, relation_lr=0.01, margin=0.1,
                           **case)
    n_ent = max(300, num_pos * (60 if cfg.comparator == "l2" else 4))
    st, batches = make_inputs(cfg, num_pos, n_ent, 2, seed=num_pos * 131 + dim, shared=(dim % 8 == 0))
    runner = to_runner(pbg, cfg, st, num_pos, 2)
    if cfg.comparator == "cos" and cfg.num_batch_negs + cfg.num_uniform_negs <= 100:  # (the largest shapes do not fit LDS)
        assert runner.route == "fused"
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs, st64 = lockstep(cfg, st, batches, keep_scores=True)
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
        sc = out.scores
        for side, pos, neg, want in ((0, sc.lhs_pos, sc.lhs_neg, out.violators_lhs),
                                     (1, sc.rhs_pos, sc.rhs_neg, out.violators_rhs)):
            ties = violator_ties(pos, neg)
            assert abs(int(runner.violators_out[k, side]) - want) <= ties, ("violators", side, k, ties)
    compare_state(cfg, runner, st, rtol, "step", st64)


def _sliced_cases():
    """Rows wider than 128 floats with at most 64 + 64 negatives: the chunk kernel takes them in slices of
    128 columns (no operator, dot / cos)."""
    import random

    rng = random.Random(5)
    cases = [
        dict(comparator="cos", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=1024),
        dict(comparator="dot", loss="softmax", num_batch_negs=50, num_uniform_negs=50, num_pos=100, dim=256),
        dict(comparator="cos", loss="logistic", num_batch_negs=64, num_uniform_negs=64, num_pos=200, dim=384),
    ]
    for _ in range(15):
        p = rng.choice([1, 3, 16, 17, 33, 48, 50, 63, 64])
        u = rng.choice([1, 5, 16, 17, 49, 50, 64])
        chunks = rng.choice([1, 2, 3])
        cases.append(dict(comparator=rng.choice(["dot", "cos"]), loss=rng.choice(["ranking", "logistic", "softmax"]),
                          num_batch_negs=p, num_uniform_negs=u, num_pos=max(1, p * chunks - rng.choice([0, 0, 1, p // 2])),
                          dim=rng.choice([256, 384, 512, 640, 2048])))
    # dims that end in a partial slice
    cases += [
        dict(comparator="cos", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=400),
        dict(comparator="dot", loss="logistic", num_batch_negs=50, num_uniform_negs=50, num_pos=75, dim=200),
        dict(comparator="cos", loss="softmax", num_batch_negs=33, num_uniform_negs=17, num_pos=66, dim=132),
        dict(comparator="cos", loss="softmax", num_batch_negs=16, num_uniform_negs=49, num_pos=40, dim=300),
        dict(comparator="dot", loss="ranking", num_batch_negs=48, num_uniform_negs=5, num_pos=100, dim=1028),
    ]
    # the two operators that act on a slice's columns alone
    for op, cmp_, loss, dim in itertools.product(("translation", "diagonal"), ("dot", "cos"), ("ranking", "softmax"), (256, 200)):
        cases.append(dict(operator=op, comparator=cmp_, loss=loss, num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=dim))
    cases.append(dict(operator="diagonal", comparator="cos", loss="logistic", num_batch_negs=17, num_uniform_negs=33, num_pos=40, dim=1024))
    # l2 (TransE at the dims the literature uses it at)
    for op, loss, dim in itertools.product(("translation", "none"), ostep.LOSS_NAMES, (200, 256)):
        cases.append(dict(operator=op, comparator="l2", loss=loss, num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=dim))
    cases += [
        dict(operator="translation", comparator="l2", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=100, dim=400),
        dict(operator="diagonal", comparator="l2", loss="softmax", num_batch_negs=33, num_uniform_negs=17, num_pos=70, dim=132),
        dict(operator="translation", comparator="l2", loss="logistic", num_batch_negs=16, num_uniform_negs=49, num_pos=40, dim=1024),
    ]
    # complex_diagonal pairs coordinate h with h + dim / 2: slices of 64 such pairs (dot; dims whose half is and is
    # not a multiple of 64, a last slice of 8 and of 4 pairs, one partial chunk)
    for loss, dim in itertools.product(ostep.LOSS_NAMES, (400, 256)):
        cases.append(dict(operator="complex_diagonal", comparator="dot", loss=loss, num_batch_negs=50, num_uniform_negs=50,
                          num_pos=130, dim=dim))
    cases += [
        dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=33, num_uniform_negs=17, num_pos=70, dim=136),
        dict(operator="complex_diagonal", comparator="dot", loss="ranking", num_batch_negs=17, num_uniform_negs=64, num_pos=40, dim=1024),
        dict(operator="complex_diagonal", comparator="dot", loss="logistic", num_batch_negs=64, num_uniform_negs=5, num_pos=100, dim=200),
        dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=48, num_uniform_negs=16, num_pos=96, dim=648),
        # ... and a single slice up to dim 128
        dict(operator="complex_diagonal", comparator="dot", loss="ranking", num_batch_negs=50, num_uniform_negs=50, num_pos=130, dim=128),
        dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=50, num_uniform_negs=50, num_pos=100, dim=64),
        dict(operator="complex_diagonal", comparator="dot", loss="logistic", num_batch_negs=17, num_uniform_negs=33, num_pos=40, dim=104),
        dict(operator="complex_diagonal", comparator="dot", loss="softmax", num_batch_negs=5, num_uniform_negs=3, num_pos=12, dim=8),
    ]
    return cases


@pytest.mark.parametrize("case", _sliced_cases(), ids=ids)
@pytest.mark.parametrize("extras", ["plain", "global_emb+weights"])
def test_sliced_chunk_kernel(pbg, case, extras):
    say("sliced", case, extras)
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    case.setdefault("operator", "none")
    cfg = ostep.StepConfig(dim=dim, dynamic=False, num_relations=2, relation_weights=[1.0, 0.5], lr=0.1,
                           relation_lr=0.01, margin=0.1, global_emb=(extras != "plain"), **case)
    workers = 3
    n_ent = max(300, num_pos * (60 if cfg.comparator == "l2" else 4))  # (l2: few repeated entities, see test_fused_kernel_shapes)
    # (l2 without operator on ONE table: an entity that is some edge's head and another's tail in a chunk scores a
    # zero distance against itself, which is rounding noise in the reference's own evaluation, model.py:215-246,
    # and the softmax spreads it over the chunk: two tables there)
    shared = num_pos % 2 == 0 and not (cfg.comparator == "l2" and cfg.operator == "none")
    st, batches = make_inputs(cfg, num_pos, n_ent, workers, seed=num_pos * 7 + dim, shared=shared)
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    if cfg.num_batch_negs + cfg.num_uniform_negs <= 100:  # (two score blocks and a slice of more rows do not fit LDS)
        assert runner.route == "fused"
    weight = None
    if extras != "plain":
        weight = torch.rand(workers, num_pos, generator=torch.Generator().manual_seed(3)) * 2
    runner.train(*pack(cfg, batches), edge_weight=None if weight is None else weight.to(DEV))
    torch.cuda.synchronize()
    # (complex_diagonal: four products per coordinate pair, whose order of rounding is the compiler's on both sides;
    # a gradient that nearly cancels then differs in its last bits, and Adagrad's division scales that up: the
    # float64 result is the anchor there as it is for l2)
    outs, st64 = lockstep(cfg, st, [b + (weight[k],) for k, b in enumerate(batches)] if weight is not None else batches,
                          keep_scores=True, anchor=cfg.operator == "complex_diagonal")
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
        sc = out.scores
        for side, pos, neg, want in ((0, sc.lhs_pos, sc.lhs_neg, out.violators_lhs),
                                     (1, sc.rhs_pos, sc.rhs_neg, out.violators_rhs)):
            ties = violator_ties(pos, neg)
            assert abs(int(runner.violators_out[k, side]) - want) <= ties, ("violators", side, k, ties)
    if st64 is not None:  # l2, complex_diagonal: the float64-anchored criterion
        compare_state(cfg, runner, st, 1e-5, "sliced", st64)
        return
    assert_close(runner.w_lhs, st.w_lhs, 1e-5, "sliced w_lhs")
    assert_close(runner.g_lhs, st.g_lhs, 1e-5, "sliced g_lhs")
    if not st.shared:
        assert_close(runner.w_rhs, st.w_rhs, 1e-5, "sliced w_rhs")
        assert_close(runner.g_rhs, st.g_rhs, 1e-5, "sliced g_rhs")
    if st.glob_lhs is not None:
        # a type's vector takes the sum of ALL the call's gradient rows: thousands of terms that largely cancel
        assert_close(runner.global_embs[0], st.glob_lhs, 1e-5, "sliced glob_lhs", atol_scale=1e-5)
        assert_close(runner.global_embs[1], st.glob_rhs, 1e-5, "sliced glob_rhs", atol_scale=1e-5)
    for name, got, want in (("rhs_op", runner.rhs_op, st.rhs_op), ("rhs_op_sum", runner.rhs_op_sum, st.rhs_op_sum)):
        for key in want:
            assert_close(got[key], want[key], 1e-5, f"sliced {name}.{key}")


def test_lockstep_training_learns_like_sequential(pbg):
    """End to end on a graph with planted structure (a ring with chords: i -> i+1,
    i -> i+7): ten passes with 1 batch per call and with 16 batches per call both
    drive the loss down by a factor of five and rank the true tail of held-out
    edges far above chance.  At an equal number of passes the lock-step run lags
    the sequential one a little (16 batches read the same tables: a larger
    effective batch), as HOGWILD workers do."""
    say("learns")
    n_ent, dim, bsz = 2000, 32, 100
    g = torch.Generator().manual_seed(0)
    src = torch.arange(n_ent).repeat(2)
    dst = torch.cat([(torch.arange(n_ent) + 1) % n_ent, (torch.arange(n_ent) + 7) % n_ent])
    perm = torch.randperm(src.shape[0], generator=g)
    src, dst = src[perm].to(DEV), dst[perm].to(DEV)
    held = 400  # held-out edges for ranking
    tr_src, tr_dst = src[held:], dst[held:]
    n_train = tr_src.shape[0] // (16 * bsz) * (16 * bsz)

    def train(workers, epochs):
        w = (torch.randn(n_ent, dim, generator=torch.Generator().manual_seed(1)) * 0.1).to(DEV)
        gs = torch.zeros(n_ent, device=DEV)
        spec = pbg.StepSpec(dim=dim, batch_size=bsz, num_workers=workers, num_batch_negs=50, num_uniform_negs=50,
                            operator="translation", comparator="dot", loss="softmax", lr=0.1)
        op = {"translation": torch.zeros(1, dim, device=DEV)}
        op_sum = {"translation": torch.zeros(1, dim, device=DEV)}
        runner = pbg.StepRunner(spec, w, gs, None, None, op, op_sum)
        rel = torch.zeros(workers, dtype=torch.int64, device=DEV)
        losses, call = [], 0
        for epoch in range(epochs):
            order = torch.randperm(n_train, generator=torch.Generator().manual_seed(100 + epoch)).to(DEV)
            total = 0.0
            for off in range(0, n_train, workers * bsz):
                idx = order[off:off + workers * bsz]
                call += 1
                runner.train(tr_src[idx].contiguous(), tr_dst[idx].contiguous(), rel, uniform_seed=call)
                total += float(runner.loss_out.sum())
            losses.append(total / n_train)
        # rank of the true rhs among 1000 uniform negatives, held-out edges
        ev = pbg.StepSpec(dim=dim, batch_size=held, num_workers=1, num_batch_negs=0, num_uniform_negs=1000,
                          operator="translation", comparator="dot", loss="softmax")
        er = pbg.StepRunner(ev, w, gs, None, None, op, op_sum)
        negs = torch.randint(0, n_ent, (1, er.spec.num_chunks, 1000), generator=torch.Generator().manual_seed(5)).to(DEV)
        _, rhs_pos, _, rhs_neg = er.forward(src[:held].contiguous(), dst[:held].contiguous(),
                                            torch.zeros(1, dtype=torch.int64, device=DEV), negs, negs)
        rank = (rhs_neg[0] >= rhs_pos[0].unsqueeze(1)).sum(1) + 1
        return losses, float(rank.float().reciprocal().mean()), float((rank <= 10).float().mean())

    seq_losses, seq_mrr, seq_h10 = train(1, 10)
    par_losses, par_mrr, par_h10 = train(16, 10)
    say("sequential", seq_losses, seq_mrr, seq_h10, "lock-step x16", par_losses, par_mrr, par_h10)
    assert seq_losses[-1] < 0.2 * seq_losses[0] and par_losses[-1] < 0.2 * par_losses[0]
    assert par_losses[-1] < 1.25 * seq_losses[-1]
    assert seq_h10 > 0.1 and par_h10 > 0.1          # chance: 10 / 1001
    assert par_mrr > 0.5 * seq_mrr


def test_lockstep_training_at_the_benchmarks_shape_learns_like_sequential(pbg):
    """The same question at the shape and staleness the benchmark line runs: cfg1's
    step (100 000 entities, dim 100, B = 1000, 50 + 50 negatives, dot, ranking with
    margin 0.1, lr 0.1, embeddings N(0, 1e-3)) on a planted graph of 1 000 000 edges
    (every entity i points at i + 1, 7, 13, ... on a ring: ten chords), trained with
    64 batches per call (16 calls per pass, every batch of a call reading the tables
    as they were when the call began) and with one batch per call (1000 calls per
    pass).  Both must drive the loss down and rank held-out true tails far above
    chance; how far the lock-step run lags at an equal number of passes is printed."""
    say("learns at cfg1's shape")
    n_ent, dim, bsz, workers = 100_000, 100, 1000, 64
    chords = torch.tensor([1, 7, 13, 29, 61, 127, 251, 509, 1021, 2039])
    src = torch.arange(n_ent).repeat_interleave(chords.numel())
    dst = (src + chords.repeat(n_ent)) % n_ent
    perm = torch.randperm(src.shape[0], generator=torch.Generator().manual_seed(0))
    src, dst = src[perm].to(DEV), dst[perm].to(DEV)
    held = 2000
    tr_src, tr_dst = src[held:], dst[held:]
    n_train = tr_src.shape[0] // (workers * bsz) * (workers * bsz)

    def train(k, epochs):
        w = (torch.randn(n_ent, dim, generator=torch.Generator().manual_seed(1)) * 1e-3).to(DEV)
        gs = torch.zeros(n_ent, device=DEV)
        spec = pbg.StepSpec(dim=dim, batch_size=bsz, num_workers=k, num_batch_negs=50, num_uniform_negs=50,
                            operator="none", comparator="dot", loss="ranking", margin=0.1, lr=0.1)
        runner = pbg.StepRunner(spec, w, gs)
        assert runner.route == "fused"
        rel = torch.zeros(k, dtype=torch.int64, device=DEV)
        losses, call = [], 0
        for epoch in range(epochs):
            order = torch.randperm(n_train, generator=torch.Generator().manual_seed(100 + epoch)).to(DEV)
            total = torch.zeros((), dtype=torch.float64, device=DEV)
            for off in range(0, n_train, k * bsz):
                idx = order[off:off + k * bsz]
                call += 1
                runner.train(tr_src[idx].contiguous(), tr_dst[idx].contiguous(), rel, uniform_seed=call)
                total += runner.loss_out.double().sum()
            losses.append(float(total) / n_train)
        # rank of the true tail among 1000 uniform negatives, held-out edges
        ev = pbg.StepSpec(dim=dim, batch_size=held, num_workers=1, num_batch_negs=0, num_uniform_negs=1000,
                          operator="none", comparator="dot", loss="ranking", margin=0.1)
        er = pbg.StepRunner(ev, w, gs)
        negs = torch.randint(0, n_ent, (1, er.spec.num_chunks, 1000), generator=torch.Generator().manual_seed(5)).to(DEV)
        _, _, _, rank, _, _ = er.ranks(src[:held].contiguous(), dst[:held].contiguous(),
                                       torch.zeros(1, dtype=torch.int64, device=DEV), negs, negs)
        rank = rank[0]
        return losses, float(rank.float().reciprocal().mean()), float((rank <= 10).float().mean())

    epochs = 8
    seq_losses, seq_mrr, seq_h10 = train(1, epochs)
    par_losses, par_mrr, par_h10 = train(workers, epochs)
    say("  sequential loss per pass", [round(x, 3) for x in seq_losses], "mrr", round(seq_mrr, 3), "hits@10", round(seq_h10, 3))
    say("  64 per call loss per pass", [round(x, 3) for x in par_losses], "mrr", round(par_mrr, 3), "hits@10", round(par_h10, 3))
    more_losses, more_mrr, more_h10 = train(workers, 2 * epochs)
    say("  64 per call, twice the passes:", [round(x, 3) for x in more_losses[epochs:]], "mrr", round(more_mrr, 3),
        "hits@10", round(more_h10, 3))
    # A fresh model pays the margin on every negative (2 sides x 100 negatives x 0.1 = 20 per edge), and Adagrad's first
    # steps of lr per coordinate overshoot from N(0, 1e-3): the first pass ends above that in both runs.
    assert seq_losses[0] < 40.0 and par_losses[0] < 40.0
    assert seq_losses[-1] < 0.01 * seq_losses[0] and par_losses[-1] < 0.01 * par_losses[0]
    assert seq_h10 > 0.1 and par_h10 > 0.1  # chance: 10 / 1001
    # 64 batches per call lag the sequential order at an equal number of passes (measured: loss 0.087 against 0.053,
    # MRR 0.076 against 0.155 after 8 passes) and keep gaining with more passes
    assert par_mrr > 0.3 * seq_mrr and par_losses[-1] < 2.5 * seq_losses[-1]
    assert more_mrr > par_mrr and more_losses[-1] < par_losses[-1]

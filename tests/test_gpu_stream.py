"""The streaming route of the training step (a chunk's positives resident in LDS,
its negatives gathered raw and streamed past them) against the oracle's lock-step
training: every operator the route takes x every loss x both relation modes, the
three row lengths it is built for, partial last chunks, the N3 regularizer,
edge weights and negatives drawn in the step."""
import itertools
import os

import pytest
import torch

from oracle import step as ostep
from tests.parity import double_state, violator_ties
from tests.test_gpu_step import DEV, compare_state, copy_of, loss_close, make_inputs, pack, say, to_runner

pytestmark = pytest.mark.gpu

CASES = []
for op, loss, dyn in itertools.product(("none", "diagonal", "complex_diagonal"), ostep.LOSS_NAMES, (False, True)):
    CASES.append(dict(operator=op, loss=loss, dynamic=dyn, num_batch_negs=50, num_uniform_negs=100, num_pos=130, dim=128))
CASES += [
    # the headline shape of the route: dim 400, chunks of 50, 1000 uniform negatives; a partial last chunk
    dict(operator="complex_diagonal", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=1000, num_pos=173,
         dim=400),
    dict(operator="complex_diagonal", loss="softmax", dynamic=True, num_batch_negs=50, num_uniform_negs=1000, num_pos=120,
         dim=400),
    dict(operator="complex_diagonal", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=300, num_pos=100,
         dim=400, shared=False),
    dict(operator="diagonal", loss="logistic", dynamic=False, num_batch_negs=50, num_uniform_negs=70, num_pos=64, dim=400),
    # dim 256; chunks of 64, 37 and 8 rows; a negatives count that is no multiple of the tile
    dict(operator="diagonal", loss="softmax", dynamic=False, num_batch_negs=64, num_uniform_negs=200, num_pos=200, dim=256),
    dict(operator="none", loss="ranking", dynamic=False, num_batch_negs=37, num_uniform_negs=91, num_pos=100, dim=256,
         shared=False),
    dict(operator="complex_diagonal", loss="logistic", dynamic=True, num_batch_negs=8, num_uniform_negs=64, num_pos=30,
         dim=256, shared=False),
    # the reference's default negatives (50 + 50, config.py:323-337) at dims beyond the LDS-resident kernel; very few negatives
    dict(operator="complex_diagonal", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=50, num_pos=173,
         dim=400),
    dict(operator="diagonal", loss="ranking", dynamic=True, num_batch_negs=50, num_uniform_negs=50, num_pos=100, dim=256),
    dict(operator="none", loss="logistic", dynamic=False, num_batch_negs=20, num_uniform_negs=8, num_pos=50, dim=400,
         shared=False),
    # dims that are no multiple of 16: the last column tile of a row is partly padding
    dict(operator="complex_diagonal", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=50, num_pos=120,
         dim=200),
    dict(operator="diagonal", loss="ranking", dynamic=True, num_batch_negs=50, num_uniform_negs=100, num_pos=100, dim=300),
    dict(operator="none", loss="logistic", dynamic=False, num_batch_negs=33, num_uniform_negs=70, num_pos=70, dim=196,
         shared=False),
    dict(operator="complex_diagonal", loss="ranking", dynamic=True, num_batch_negs=50, num_uniform_negs=200, num_pos=130,
         dim=292, regularization_coef=0.02),
    dict(operator="diagonal", loss="softmax", dynamic=False, num_batch_negs=64, num_uniform_negs=40, num_pos=128, dim=208),
    # fewer positives than a chunk holds; a single positive
    dict(operator="diagonal", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=100, num_pos=30, dim=128),
    dict(operator="complex_diagonal", loss="ranking", dynamic=True, num_batch_negs=50, num_uniform_negs=64, num_pos=1, dim=256),
    # no batch negatives: the chunk is as long as the uniform draw (model.py:648-650)
    dict(operator="diagonal", loss="softmax", dynamic=False, num_batch_negs=0, num_uniform_negs=64, num_pos=150, dim=128),
    dict(operator="none", loss="logistic", dynamic=True, num_batch_negs=0, num_uniform_negs=64, num_pos=64, dim=256),
    # the N3 regularizer (regularizers.py:51-97); the first is the reference's FB15k example
    # (examples/configs/fb15k_config_cpu.py: ComplEx, one relation per edge, 1000 uniform negatives, coefficient 1e-3)
    dict(operator="complex_diagonal", loss="softmax", dynamic=True, num_batch_negs=50, num_uniform_negs=1000, num_pos=120,
         dim=400, regularization_coef=1e-3),
    dict(operator="complex_diagonal", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=100, num_pos=130,
         dim=128, regularization_coef=0.05),
    dict(operator="diagonal", loss="logistic", dynamic=False, num_batch_negs=37, num_uniform_negs=91, num_pos=100, dim=256,
         regularization_coef=0.02, shared=False),
    dict(operator="diagonal", loss="softmax", dynamic=True, num_batch_negs=50, num_uniform_negs=100, num_pos=130, dim=128,
         regularization_coef=0.05),
    dict(operator="none", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=100, num_pos=130, dim=128,
         regularization_coef=0.05),
    dict(operator="none", loss="ranking", dynamic=True, num_batch_negs=0, num_uniform_negs=64, num_pos=70, dim=128,
         regularization_coef=0.05),
]


# The cos comparator (the reference's default, config.py:185-190) without an operator: the same kernels on a
# normalised copy of the tables, the normalisation's backward in the update.  The three update kernels each
# have that path: rows of up to 128 floats, wider rows, and a wave per table row where gradient rows
# outnumber table rows 32 to 1; with 3 batches per call and 600 negatives per chunk on 300 entities a row
# has more positions than one look at the sorted keys shows.
COS_CASES = []
for loss, dyn in itertools.product(ostep.LOSS_NAMES, (False, True)):
    COS_CASES.append(dict(comparator="cos", operator="none", loss=loss, dynamic=dyn, num_batch_negs=50, num_uniform_negs=300,
                          num_pos=130, dim=128))
COS_CASES += [
    dict(comparator="cos", operator="none", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=1000,
         num_pos=173, dim=400),
    dict(comparator="cos", operator="none", loss="ranking", dynamic=False, num_batch_negs=37, num_uniform_negs=291,
         num_pos=100, dim=256, shared=False),
    dict(comparator="cos", operator="none", loss="logistic", dynamic=True, num_batch_negs=50, num_uniform_negs=300,
         num_pos=120, dim=200),
    dict(comparator="cos", operator="none", loss="softmax", dynamic=False, num_batch_negs=0, num_uniform_negs=64,
         num_pos=150, dim=128),
    dict(comparator="cos", operator="none", loss="ranking", dynamic=False, num_batch_negs=50, num_uniform_negs=600,
         num_pos=60, dim=128),
    dict(comparator="cos", operator="none", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=1000,
         num_pos=60, dim=256),
    dict(comparator="cos", operator="none", loss="logistic", dynamic=False, num_batch_negs=50, num_uniform_negs=1000,
         num_pos=60, dim=128, shared=False),
]
CASES += COS_CASES


def ids(case):
    return "-".join(f"{v}" for v in case.values())


def lockstep64(cfg, st, batches, keep_scores=False):
    """oracle.step.train_lockstep on `st` and on a float64 copy of it.  A row that is
    a negative of many chunks sums hundreds of gradient terms of mixed sign, and a
    score row of a thousand negatives sums a thousand exponentials: the CPU path's own
    fp32 result then lies further from the exact one than the tolerance (3e-5 against
    1e-5 at dim 400 with 1000 negatives), so the float64 result anchors the comparison
    (tests.parity.anchored_close)."""
    st64 = double_state(st)
    outs = ostep.train_lockstep(cfg, st, batches, keep_scores=keep_scores)
    for out, exact in zip(outs, ostep.train_lockstep(cfg, st64, batches)):
        out.exact_loss = exact.loss
    return outs, st64


@pytest.fixture(autouse=True)
def _keep_to_the_streaming_kernels(monkeypatch):
    """A shape without operator whose chunk has at most about 100 negatives is taken by the chunk kernel on
    slices first; these tests are about the streaming kernels."""
    monkeypatch.setenv("PBG_DISABLE_SLICED", "1")


def build(pbg, case, workers, seed_shift=0):
    case = dict(case)
    num_pos, dim = case.pop("num_pos"), case.pop("dim")
    shared = case.pop("shared", True)
    cfg = ostep.StepConfig(dim=dim, comparator=case.pop("comparator", "dot"), num_relations=3,
                           relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01, margin=0.1, **case)
    st, batches = make_inputs(cfg, num_pos, max(300, num_pos * 4), workers, seed=num_pos + dim + seed_shift, shared=shared)
    return cfg, st, batches, num_pos


@pytest.mark.parametrize("case", CASES, ids=ids)
@pytest.mark.parametrize("workers", [1, 3])
def test_stream_route_matches_the_oracle(pbg, case, workers):
    say("stream", case, workers)
    cfg, st, batches, num_pos = build(pbg, case, workers)
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    assert runner.route == "stream"
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs, st64 = lockstep64(cfg, st, batches, keep_scores=True)
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
        sc = out.scores
        for side, pos, neg, want in ((0, sc.lhs_pos, sc.lhs_neg, out.violators_lhs),
                                     (1, sc.rhs_pos, sc.rhs_neg, out.violators_rhs)):
            ties = violator_ties(pos, neg)
            assert abs(int(runner.violators_out[k, side]) - want) <= ties, ("violators", side, k, ties)
        if cfg.regularization_coef:
            assert out.reg > 0.0 and float(runner.reg_out[k]) == pytest.approx(out.reg, rel=1e-5), ("reg", k)
    compare_state(cfg, runner, st, 1e-5, "stream", st64)


@pytest.mark.parametrize("case", [CASES[0], CASES[5], CASES[18], CASES[23], COS_CASES[0], COS_CASES[7]], ids=ids)
def test_stream_route_with_edge_weights(pbg, case):
    say("stream+weights", case)
    cfg, st, batches, num_pos = build(pbg, case, 2)
    g = torch.Generator().manual_seed(7)
    weights = [0.25 + 2.0 * torch.rand(num_pos, generator=g) for _ in batches]
    weights[0][::5] = 0.0
    unweighted = copy_of(st)
    runner = to_runner(pbg, cfg, st, num_pos, 2)
    assert runner.route == "stream"
    runner.train(*pack(cfg, batches), edge_weight=torch.stack(weights).to(DEV))
    torch.cuda.synchronize()
    outs, st64 = lockstep64(cfg, st, [b + (w,) for b, w in zip(batches, weights)])
    ostep.train_lockstep(cfg, unweighted, batches)
    for k, out in enumerate(outs):
        assert loss_close(float(runner.loss_out[k]), out), ("loss", k, float(runner.loss_out[k]), out.loss)
    compare_state(cfg, runner, st, 1e-5, "stream+weights", st64)
    assert (st.w_lhs - unweighted.w_lhs).abs().max() > 1e-3 * st.w_lhs.abs().max()


@pytest.mark.parametrize("case", [CASES[3], CASES[19], COS_CASES[6]], ids=ids)
def test_stream_route_draws_its_negatives(pbg, case):
    """A call that draws its uniform negatives from a seed equals, bit for bit, the call
    that is handed the same draw."""
    say("stream, in-step negatives", case)
    from pytorch_biggraph_amd import native

    cfg, st, batches, num_pos = build(pbg, case, 3)
    lhs, rhs, rel, _, _ = pack(cfg, batches)
    a = to_runner(pbg, cfg, st, num_pos, 3)
    b = to_runner(pbg, cfg, st, num_pos, 3)
    assert a.route == "stream"
    seed = 0x0FEDCBA987654321
    shape = (3, a.spec.num_chunks, cfg.num_uniform_negs)
    ul = native.sample_uniform_negatives(seed, 0, st.w_lhs.shape[0], shape, DEV)
    ur = native.sample_uniform_negatives(seed, 1, st.w_rhs.shape[0], shape, DEV)
    a.train(lhs, rhs, rel, ul, ur)
    b.train(lhs, rhs, rel, uniform_seed=seed)
    torch.cuda.synchronize()
    assert torch.equal(a.loss_out, b.loss_out) and torch.equal(a.violators_out, b.violators_out)
    assert torch.equal(a.w_lhs, b.w_lhs) and torch.equal(a.g_lhs, b.g_lhs)
    for k in a.rhs_op:
        assert torch.equal(a.rhs_op[k], b.rhs_op[k])


def test_twenty_calls_on_the_stream_route(pbg):
    """20 training calls of 2 batches each, the state carried from call to call."""
    case = dict(operator="complex_diagonal", loss="softmax", dynamic=False, num_batch_negs=50, num_uniform_negs=200, num_pos=100,
                dim=128)
    say("stream, 20 calls", case)
    cfg, st, _, num_pos = build(pbg, case, 2)
    runner = to_runner(pbg, cfg, st, num_pos, 2)
    assert runner.route == "stream"
    st64 = double_state(st)
    for call in range(20):
        _, batches = make_inputs(cfg, num_pos, st.w_lhs.shape[0], 2, seed=1000 + call, shared=True)
        runner.train(*pack(cfg, batches))
        ostep.train_lockstep(cfg, st, batches)
        ostep.train_lockstep(cfg, st64, batches)
    torch.cuda.synchronize()
    compare_state(cfg, runner, st, 1e-4, "stream x20", st64)  # 1e-4 after many steps

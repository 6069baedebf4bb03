"""Random combinations of the step's options (operator, comparator, relation mode,
negatives, bias, all_negs, global embeddings, max_norm, regularizer, tables, K)
against the oracle: the forward's scores, then one lock-step training call.

The loss is the logistic one throughout: it has no hinge (two correct fp32
evaluations can take different sides of a hinge for good) and it sees a common
shift of scores (ranking and softmax do not, which leaves some parameters with
an exactly zero gradient whose rounding noise Adagrad turns into full steps)."""
import random

import pytest
import torch

from oracle import step as ostep
from tests.test_gpu_step import compare_scores, compare_state, lockstep, make_inputs, pack, say, to_runner

pytestmark = pytest.mark.gpu


def sample_case(rng, wide=False):
    """wide: also bias with l2 and bias with the regularizer."""
    op = rng.choice(ostep.OPERATOR_NAMES)
    cmp_ = rng.choice(ostep.COMPARATOR_NAMES)
    dyn = rng.random() < 0.4
    bias = rng.random() < (0.5 if wide else 0.3) and (wide or cmp_ != "l2")
    glob = (not dyn) and rng.random() < 0.3
    reg = 0.02 if (rng.random() < (0.4 if wide else 0.2) and op not in ("linear", "affine", "none") and (wide or not bias)) else 0.0
    dim = rng.choice([6, 8, 12, 16, 24, 32, 100, 128])
    nb, nu = rng.choice([0, 4, 10, 50]), rng.choice([0, 3, 10, 50])
    if nb == 0 and nu == 0:
        nu = 5
    dl = rng.random() < 0.15
    shared = rng.random() < 0.6
    if glob and cmp_ in ("l2", "squared_l2"):
        shared = False  # (a distance between two rows of one type does not depend on the type's vector)
    return dict(dim=dim, operator=op, comparator=cmp_, loss="logistic", dynamic=dyn, num_batch_negs=nb, num_uniform_negs=nu,
                disable_lhs_negs=dl, disable_rhs_negs=(not dl) and rng.random() < 0.15, bias=bias,
                all_negs=rng.random() < 0.25, global_emb=glob, max_norm=(0.3 * dim ** 0.5 if rng.random() < 0.3 else None),
                regularization_coef=reg), dict(num_pos=rng.choice([7, 20, 33, 50, 64, 130]), shared=shared,
                                               workers=rng.choice([1, 1, 2, 3]))


def cases():
    rng = random.Random(20240607)
    first = [sample_case(rng) for _ in range(120)]
    rng = random.Random(20241125)
    return first + [sample_case(rng, wide=True) for _ in range(40)]


@pytest.mark.parametrize("index", range(160))
def test_random_combination(pbg, index):
    kw, extra = cases()[index]
    say("combination", index, kw, extra)
    cfg = ostep.StepConfig(num_relations=3, relation_weights=[1.0, 0.5, 2.0], lr=0.1, relation_lr=0.01, margin=0.1, **kw)
    num_pos, workers = extra["num_pos"], extra["workers"]
    st, batches = make_inputs(cfg, num_pos, 1500 if cfg.comparator == "l2" else 200, workers, seed=index,
                              shared=extra["shared"], scale=0.3)
    runner = to_runner(pbg, cfg, st, num_pos, workers)
    got = runner.forward(*pack(cfg, batches))
    for k, b in enumerate(batches):
        want, _ = ostep.forward_backward(cfg, st, *b, keep_scores=True)
        compare_scores(cfg, tuple(t[k] for t in got), want.scores)
    runner.train(*pack(cfg, batches))
    torch.cuda.synchronize()
    outs, st64 = lockstep(cfg, st, batches)
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert float(runner.loss_out[k]) == pytest.approx(out.loss, rel=rtol, abs=1e-5), ("loss", k)
    compare_state(cfg, runner, st, rtol, "combination", st64)

"""Pins the oracle's global embeddings (model.py:433-441,486-492): adding the
type's vector to every gathered row is the same as shifting the table, and the
vector's gradient is the sum of the rows' gradients."""
import pytest
import torch

from oracle import step as ostep


def _case(operator="complex_diagonal", comparator="dot", shared=True, seed=0):
    cfg = ostep.StepConfig(dim=8, operator=operator, comparator=comparator, loss="softmax", num_batch_negs=5,
                           num_uniform_negs=4, num_relations=2, relation_weights=[1.0, 0.7], global_emb=True,
                           lr=0.1, relation_lr=0.05)
    g = torch.Generator().manual_seed(seed)
    w_l = torch.randn(40, 8, generator=g) * 0.5
    w_r = None if shared else torch.randn(45, 8, generator=g) * 0.5
    st = ostep.make_state(cfg, w_l, w_r)
    for d in (st.rhs_op,):
        for k in d:
            d[k] = d[k] + 0.2 * torch.randn(d[k].shape, generator=g)
    st.glob_lhs += 0.3 * torch.randn(8, generator=g)
    if not shared:
        st.glob_rhs += 0.3 * torch.randn(8, generator=g)
    n_r = 40 if shared else 45
    lhs, rhs = torch.randint(0, 40, (13,), generator=g), torch.randint(0, n_r, (13,), generator=g)
    ul, ur = torch.randint(0, 40, (3, 4), generator=g), torch.randint(0, n_r, (3, 4), generator=g)
    return cfg, st, lhs, rhs, 1, ul, ur


def test_state_starts_at_zero_and_is_shared_with_the_type():
    cfg = ostep.StepConfig(dim=4, global_emb=True)
    st = ostep.make_state(cfg, torch.zeros(3, 4))
    assert st.glob_lhs is st.glob_rhs and float(st.glob_lhs.abs().sum()) == 0.0
    st2 = ostep.make_state(cfg, torch.zeros(3, 4), torch.zeros(5, 4))
    assert st2.glob_lhs is not st2.glob_rhs
    assert ostep.make_state(ostep.StepConfig(dim=4), torch.zeros(3, 4)).glob_lhs is None


@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("operator,comparator", [("complex_diagonal", "dot"), ("translation", "l2"), ("none", "cos")])
def test_scores_equal_those_of_the_shifted_tables(operator, comparator, shared):
    cfg, st, lhs, rhs, rel, ul, ur = _case(operator, comparator, shared)
    out, _ = ostep.forward_backward(cfg, st, lhs, rhs, rel, ul, ur, keep_scores=True)
    plain = ostep.StepConfig(**{**cfg.__dict__, "global_emb": False})
    st2 = ostep.make_state(plain, st.w_lhs + st.glob_lhs, None if shared else st.w_rhs + st.glob_rhs)
    st2.rhs_op = st.rhs_op
    out2, _ = ostep.forward_backward(plain, st2, lhs, rhs, rel, ul, ur, keep_scores=True)
    for a, b in zip((out.scores.lhs_pos, out.scores.rhs_pos, out.scores.lhs_neg, out.scores.rhs_neg),
                    (out2.scores.lhs_pos, out2.scores.rhs_pos, out2.scores.lhs_neg, out2.scores.rhs_neg)):
        assert torch.allclose(a, b, rtol=1e-6, atol=1e-6)
    assert out.loss == pytest.approx(out2.loss, rel=1e-6)


@pytest.mark.parametrize("shared", [True, False])
def test_gradient_is_the_sum_of_the_row_gradients_and_the_step_is_adagrad(shared):
    cfg, st, lhs, rhs, rel, ul, ur = _case(shared=shared)
    _, grads = ostep.forward_backward(cfg, st, lhs, rhs, rel, ul, ur)
    rows_l = grads.sparse_lhs.to_dense().sum(0)
    if shared:
        assert grads.glob_rhs is None
        assert torch.allclose(grads.glob_lhs, rows_l, rtol=1e-5, atol=1e-6)
    else:
        assert torch.allclose(grads.glob_lhs, rows_l, rtol=1e-5, atol=1e-6)
        assert torch.allclose(grads.glob_rhs, grads.sparse_rhs.to_dense().sum(0), rtol=1e-5, atol=1e-6)
    before, g = st.glob_lhs.clone(), grads.glob_lhs
    ostep.apply_grads(cfg, st, grads)
    # AsyncAdagrad from a zero sum with the relation learning rate: p -= lr g / (|g| + 1e-10)
    assert torch.allclose(st.glob_lhs, before - 0.05 * g / (g.abs() + 1e-10), rtol=1e-5, atol=1e-7)
    assert torch.allclose(st.glob_lhs_sum, g * g, rtol=1e-6)


def test_dynamic_relations_refuse_global_embeddings():
    cfg = ostep.StepConfig(dim=4, dynamic=True, num_relations=2, relation_weights=[1.0, 1.0], num_batch_negs=2,
                           num_uniform_negs=0)
    w = torch.randn(6, 4)
    with pytest.raises(RuntimeError, match="Cannot have global embs with dynamic rels"):
        ostep.model_forward(cfg, w[:3], w[3:], None, None, torch.tensor([0, 1, 0]), None, None, torch.zeros(4), torch.zeros(4))

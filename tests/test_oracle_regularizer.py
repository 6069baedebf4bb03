"""Pins the oracle's N3 regularizer (regularizers.py:51-97) to independent
formulations: complex arithmetic in numpy, closed forms, finite differences."""
import numpy as np
import pytest
import torch

from oracle import step as ostep


def _setup(operator, dynamic, num_pos=130, dim=8, nrel=3, comparator="dot", seed=0):
    cfg = ostep.StepConfig(dim=dim, operator=operator, comparator=comparator, loss="softmax", num_batch_negs=50,
                           num_uniform_negs=0, dynamic=dynamic, num_relations=nrel, relation_weights=[1.0] * nrel,
                           regularization_coef=1e-2)
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(60, dim, generator=g, dtype=torch.float64)
    st = ostep.make_state(cfg, w)
    for d in (st.lhs_op, st.rhs_op):
        for k in d:
            d[k] = (d[k] + 0.3 * torch.randn(d[k].shape, generator=g)).double()
    lhs = torch.randint(0, 60, (num_pos,), generator=g)
    rhs = torch.randint(0, 60, (num_pos,), generator=g)
    rel = torch.randint(0, nrel, (num_pos,), generator=g) if dynamic else 1
    return cfg, st, lhs, rhs, rel


def _reg(cfg, st, lhs, rhs, rel):
    sc = ostep.model_forward(cfg, st.w_lhs[lhs], st.w_rhs[rhs], None, None, rel, st.lhs_op or None, st.rhs_op or None)
    return sc.reg


def test_none_operator_is_the_sum_of_cubed_magnitudes():
    cfg, st, lhs, rhs, rel = _setup("none", False)
    want = 1e-2 * float((st.w_lhs[lhs].abs() ** 3).sum() + (st.w_lhs[rhs].abs() ** 3).sum())
    assert float(_reg(cfg, st, lhs, rhs, rel)) == pytest.approx(want, rel=1e-12)
    # no regularizer, no value (model.py:845-846)
    cfg.regularization_coef = 0.0
    assert _reg(cfg, st, lhs, rhs, rel) is None


@pytest.mark.parametrize("operator", ["diagonal", "translation"])
def test_static_elementwise_operators(operator):
    """|op(x)|^3 on the operated side, |x|^3 on the other, and |p|^3 once per CHUNK
    (len(src_pos) of the chunked positives, regularizers.py:91-93): 130 edges in
    chunks of 50 are 3 chunks."""
    cfg, st, lhs, rhs, rel = _setup(operator, False)
    p = st.rhs_op[operator][rel]
    x = st.w_lhs[rhs]
    y = x * p if operator == "diagonal" else x + p
    want = 1e-2 * float((st.w_lhs[lhs].abs() ** 3).sum() + (y.abs() ** 3).sum() + 3 * (p.abs() ** 3).sum())
    assert float(_reg(cfg, st, lhs, rhs, rel)) == pytest.approx(want, rel=1e-12)


def test_static_complex_diagonal_against_numpy_complex():
    """The halves of a row are the real and imaginary parts (operators.py:139-149):
    with z = x_re + i x_im and q = p_re + i p_im the regularizer is
    coef * (sum |z_lhs|^3 + sum |z_rhs q|^3 + chunks * sum |q|^3)."""
    cfg, st, lhs, rhs, rel = _setup("complex_diagonal", False)
    h = cfg.dim // 2
    z = lambda t: t[..., :h].numpy() + 1j * t[..., h:].numpy()
    q = st.rhs_op["real"][rel].numpy() + 1j * st.rhs_op["imag"][rel].numpy()
    want = 1e-2 * (np.sum(np.abs(z(st.w_lhs[lhs])) ** 3) + np.sum(np.abs(z(st.w_lhs[rhs]) * q) ** 3)
                   + 3 * np.sum(np.abs(q) ** 3))
    assert float(_reg(cfg, st, lhs, rhs, rel)) == pytest.approx(want, rel=1e-12)


def test_dynamic_complex_diagonal_is_both_directions():
    """model.py:721-758: the forward edges regularize (lhs, op_rhs(rhs)) with the rhs
    operators of the edges' relations, the reverse edges (rhs, op_lhs(lhs)) with the
    lhs operators; the parameters enter once per EDGE (regularizers.py:73-76)."""
    cfg, st, lhs, rhs, rel = _setup("complex_diagonal", True)
    h = cfg.dim // 2
    z = lambda t: t[..., :h].numpy() + 1j * t[..., h:].numpy()
    total = 0.0
    for src, dst, ops in ((lhs, rhs, st.rhs_op), (rhs, lhs, st.lhs_op)):
        q = ops["real"][rel].numpy() + 1j * ops["imag"][rel].numpy()  # [B, h]
        total += np.sum(np.abs(z(st.w_lhs[src])) ** 3) + np.sum(np.abs(z(st.w_lhs[dst]) * q) ** 3) + np.sum(np.abs(q) ** 3)
    assert float(_reg(cfg, st, lhs, rhs, rel)) == pytest.approx(1e-2 * total, rel=1e-12)


def test_cos_comparator_regularizes_the_normalised_rows():
    """The regularizer sees what adjust_embs returns, i.e. rows after
    comparator.prepare (model.py:501-502,784-785)."""
    cfg, st, lhs, rhs, rel = _setup("none", False, comparator="cos")
    unit = lambda x: x / x.norm(2, dim=-1, keepdim=True)
    want = 1e-2 * float((unit(st.w_lhs[lhs]).abs() ** 3).sum() + (unit(st.w_lhs[rhs]).abs() ** 3).sum())
    assert float(_reg(cfg, st, lhs, rhs, rel)) == pytest.approx(want, rel=1e-10)


def test_linear_operator_has_no_regularizer():
    cfg, st, lhs, rhs, rel = _setup("linear", False)
    with pytest.raises(NotImplementedError):
        _reg(cfg, st, lhs, rhs, rel)


@pytest.mark.parametrize("operator,dynamic", [("complex_diagonal", False), ("diagonal", True), ("translation", False)])
def test_step_gradient_includes_the_regularizer(operator, dynamic):
    """(loss + reg).backward() (train_cpu.py:102-103): the gradient the step applies
    differs from the unregularized one by d reg / d theta, checked by central
    differences of the regularizer alone."""
    cfg, st, lhs, rhs, rel = _setup(operator, dynamic, num_pos=20, dim=6)
    cfg.regularization_coef = 1.0  # large against the fp32 rounding of the loss gradient it is separated from
    st.w_lhs = st.w_lhs.float()
    st.w_rhs = st.w_lhs
    for d in (st.lhs_op, st.rhs_op):
        for k in d:
            d[k] = d[k].float()
    out, grads = ostep.forward_backward(cfg, st, lhs, rhs, rel, None, None)
    cfg0 = ostep.StepConfig(**{**cfg.__dict__, "regularization_coef": 0.0})
    out0, grads0 = ostep.forward_backward(cfg0, st, lhs, rhs, rel, None, None)
    assert out.loss == pytest.approx(out0.loss, rel=1e-6) and out0.reg == 0.0 and out.reg > 0.0
    d_w = (grads.sparse_lhs.to_dense() - grads0.sparse_lhs.to_dense()).double()

    def reg_at(w64, ops64):
        s2 = ostep.TrainState(w_lhs=w64, g_lhs=st.g_lhs, w_rhs=w64, g_rhs=st.g_lhs, lhs_op=ops64[0], rhs_op=ops64[1])
        return float(_reg(cfg, s2, lhs, rhs, rel))

    w64 = st.w_lhs.double()
    ops64 = [{k: v.double() for k, v in d.items()} for d in (st.lhs_op, st.rhs_op)]
    assert out.reg == pytest.approx(reg_at(w64, ops64), rel=1e-5)
    eps = 1e-6
    for row, col in ((int(lhs[0]), 1), (int(rhs[3]), 4), (int(rhs[7]), 0)):
        wp, wm = w64.clone(), w64.clone()
        wp[row, col] += eps
        wm[row, col] -= eps
        fd = (reg_at(wp, ops64) - reg_at(wm, ops64)) / (2 * eps)
        assert float(d_w[row, col]) == pytest.approx(fd, rel=1e-3, abs=2e-6)
    name = next(iter(st.rhs_op))
    d_p = (grads.rhs_op[name] - grads0.rhs_op[name]).double()
    r = int(rel[0]) if dynamic else rel
    for col in (0, 2):
        plus = [dict(ops64[0]), {k: v.clone() for k, v in ops64[1].items()}]
        minus = [dict(ops64[0]), {k: v.clone() for k, v in ops64[1].items()}]
        plus[1][name][r, col] += eps
        minus[1][name][r, col] -= eps
        fd = (reg_at(w64, plus) - reg_at(w64, minus)) / (2 * eps)
        assert float(d_p[r, col]) == pytest.approx(fd, rel=1e-3, abs=2e-6)

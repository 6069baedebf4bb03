"""What pins the oracle's half_precision path (oracle.step, model.py:504-505,827-829).
The reference only casts on a CUDA device and its tests hold no vector for the
switch, so the oracle is checked against what the arithmetic fixes: inputs whose
every intermediate is a float16 number must give the fp32 path's result bit for
bit, and on a small random case each rounding point is restated with numpy float16
(which a missing or an extra cast fails: a positive score rounded to float16,
negative scores or table gradients that are not float16 numbers, a term left out)."""
import numpy as np
import pytest
import torch

from oracle import step as ostep


def dyadic_state(cfg, n_ent, seed):
    """Rows whose entries are multiples of 1/8 in [-1, 1]: with dim 6 every product,
    score (|s| <= 6, multiples of 1/64) and gradient entry below is a float16 number."""
    g = torch.Generator().manual_seed(seed)
    w = torch.randint(-8, 9, (n_ent, cfg.dim), generator=g).float() / 8
    return ostep.make_state(cfg, w, None)


def batches_for(cfg, num_pos, n_ent, workers, seed):
    g = torch.Generator().manual_seed(seed)
    _, c, _ = cfg.chunking(num_pos)
    out = []
    for _ in range(workers):
        out.append((torch.randint(0, n_ent, (num_pos,), generator=g), torch.randint(0, n_ent, (num_pos,), generator=g), 0,
                    torch.randint(0, n_ent, (c, cfg.num_uniform_negs), generator=g),
                    torch.randint(0, n_ent, (c, cfg.num_uniform_negs), generator=g)))
    return out


@pytest.mark.parametrize("operator", ["none", "translation"])
def test_exact_inputs_give_the_fp32_result(operator):
    kw = dict(dim=6, operator=operator, comparator="dot", loss="ranking", margin=0.125, num_batch_negs=4, num_uniform_negs=3,
              relation_weights=[1.0], lr=0.1)
    full, half = ostep.StepConfig(**kw), ostep.StepConfig(half_precision=True, **kw)
    st_a, st_b = dyadic_state(full, 40, 1), dyadic_state(half, 40, 1)
    for st in (st_a, st_b):
        for k in st.rhs_op:  # translation by multiples of 1/8 as well
            st.rhs_op[k] = torch.randint(-4, 5, st.rhs_op[k].shape, generator=torch.Generator().manual_seed(2)).float() / 8
    batches = batches_for(full, 10, 40, 2, 3)
    outs_a = ostep.train_lockstep(full, st_a, batches, keep_scores=True)
    outs_b = ostep.train_lockstep(half, st_b, batches, keep_scores=True)
    for a, b in zip(outs_a, outs_b):
        assert a.loss == b.loss
        for name in ("lhs_pos", "rhs_pos", "lhs_neg", "rhs_neg"):
            assert torch.equal(getattr(a.scores, name), getattr(b.scores, name)), name
    assert torch.equal(st_a.w_lhs, st_b.w_lhs) and torch.equal(st_a.g_lhs, st_b.g_lhs)
    for k in st_a.rhs_op:
        assert torch.equal(st_a.rhs_op[k], st_b.rhs_op[k])


def h(x):
    """float16 rounding of an fp32 / fp64 array, returned as float64"""
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float64)


def test_rounding_points_restated_with_numpy_float16():
    """One chunk, dot comparator (prepare is the identity, so the gradient of a table
    row IS the gradient of its float16 copy), logistic loss, batch + uniform negatives."""
    cfg = ostep.StepConfig(dim=5, comparator="dot", loss="logistic", num_batch_negs=4, num_uniform_negs=3,
                           half_precision=True, relation_weights=[1.0])
    g = torch.Generator().manual_seed(7)
    n_ent, p, u = 30, 4, 3
    w = torch.randn(n_ent, cfg.dim, generator=g)
    st = ostep.make_state(cfg, w, None)
    lhs = torch.tensor([0, 1, 2, 3])
    rhs = torch.tensor([4, 5, 6, 7])
    ul = torch.tensor([[8, 9, 10]])
    ur = torch.tensor([[11, 12, 13]])  # every row once: a table row's gradient is one prepared row's
    out, grads = ostep.forward_backward(cfg, st, lhs, rhs, 0, ul, ur, keep_scores=True)

    w16 = h(w.numpy())
    L, R = w16[lhs.numpy()], w16[rhs.numpy()]
    ln = np.concatenate([L, w16[ul[0].numpy()]])  # [p + u, D]
    rn = np.concatenate([R, w16[ur[0].numpy()]])
    pos = (L.astype(np.float32) * R.astype(np.float32)).sum(-1, dtype=np.float32)  # fp32, NOT rounded (model.py:177)
    s_l, s_r = h(R @ ln.T), h(L @ rn.T)  # float16 products (model.py:179-180)
    assert np.allclose(out.scores.lhs_pos.numpy(), pos, rtol=1e-6, atol=1e-7)
    ulp = lambda x: 2.0 ** (np.floor(np.log2(np.maximum(np.abs(x), 2.0 ** -14))) - 10)
    mask = np.zeros((p, p + u), dtype=bool)
    mask[np.arange(p), np.arange(p)] = True
    got_l, got_r = out.scores.lhs_neg.numpy().astype(np.float64), out.scores.rhs_neg.numpy().astype(np.float64)
    assert (got_l[mask] == -1e9).all() and (got_r[mask] == -1e9).all()
    assert (np.abs(got_l - s_l)[~mask] <= ulp(s_l)[~mask]).all() and (np.abs(got_r - s_r)[~mask] <= ulp(s_r)[~mask]).all()
    # values that ARE float16 numbers (an unrounded product would not be)
    assert (h(got_l[~mask]) == got_l[~mask]).all()

    # logistic loss (losses.py:85-114): dLoss/dneg = sigmoid(neg) / N, dLoss/dpos = sigmoid(pos) - 1 per side
    sig = lambda x: 1.0 / (1.0 + np.exp(-np.maximum(x, -80.0)))
    n = p + u
    d_l = np.where(mask, 0.0, sig(got_l) / n)
    d_r = np.where(mask, 0.0, sig(got_r) / n)
    dpos = 2.0 * (sig(pos.astype(np.float64)) - 1.0)
    d_l16, d_r16 = h(d_l), h(d_r)  # the cast's backward (model.py:827-829)
    # gradient of lhs positive i: positive pair, its row of S_R as the left operand, its column of S_L as a negative
    terms = [h(dpos[:, None] * R), h(d_r16 @ rn), h(d_l16.T @ R)[:p]]
    want = terms[0] + terms[1] + terms[2]
    got = grads.sparse_lhs.coalesce().to_dense().double()  # one table: it carries both sides' rows
    got_rows = got[lhs].numpy()
    # each term is a float16 number and so is every partial sum: two roundings of at most one ulp each
    bound = 2.5 * ulp(np.abs(want) + np.abs(terms[0]) + np.abs(terms[1]) + np.abs(terms[2]))
    assert (np.abs(got_rows - want) <= bound).all(), np.abs(got_rows - want).max()
    assert (h(got_rows) == got_rows).all()  # the table gradient is made of float16 numbers
    # a uniform negative of the lhs side: only its column of S_L
    got_u = got[ul[0]].numpy()
    want_u = h(d_l16.T @ R)[p:]
    assert (np.abs(got_u - want_u) <= ulp(want_u)).all()

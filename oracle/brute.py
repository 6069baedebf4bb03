"""Per-edge float64 restatement of the scoring rules (test infrastructure only).

Independent of ``oracle.step``: no chunk tensors, no bmm, no mask index
arithmetic.  It states what the reference's docs say a score IS
(docs/source/batch_preparation.rst, scoring.rst; model.py:508-580,666-758):

* an edge e = (u, r, v) sits in chunk c = e // P at position i = e % P;
* its left-hand negatives are the left-hand entities of the other edges of
  its chunk, then the chunk's U uniformly sampled entities; likewise on the
  right; the pair with itself, and with the padding positions of an incomplete
  last chunk, is masked with -1e9;
* standard mode scores (u', r, v) as k(f(u'), f(op_r(v))) and (u, r, v') as
  k(f(u), f(op_r(v')));
* dynamic mode scores (u', r, v) as k(f(u'), f(op^rhs_r(v))) and (u, r, v') as
  k(f(op^lhs_r(u)), f(v')), the positive once per direction.
"""
import math
from typing import Dict, Optional

import numpy as np


def _op(name: str, x: np.ndarray, params: Optional[Dict[str, np.ndarray]], r: int) -> np.ndarray:
    if params is None or name == "none":
        return x
    if name == "diagonal":
        return params["diagonal"][r] * x
    if name == "translation":
        return x + params["translation"][r]
    if name == "linear":
        return params["linear_transformation"][r] @ x
    if name == "affine":
        return params["linear_transformation"][r] @ x + params["translation"][r]
    if name == "complex_diagonal":
        h = x.shape[0] // 2
        a = x[:h] + 1j * x[h:]
        b = params["real"][r] + 1j * params["imag"][r]
        y = a * b
        return np.concatenate([y.real, y.imag])
    raise NotImplementedError(name)


def _prep(comparator: str, x: np.ndarray, bias: bool = False) -> np.ndarray:
    if bias:  # the first coordinate is the row's bias and stays as it is (model.py:311-314)
        return np.concatenate([x[:1], _prep(comparator, x[1:])])
    if comparator == "cos":
        return x / math.sqrt(float(x @ x))
    return x


def _kappa(comparator: str, a: np.ndarray, b: np.ndarray, bias: bool = False) -> float:
    if bias:  # score of the remaining coordinates plus both rows' biases (model.py:328-342)
        return _kappa(comparator, a[1:], b[1:]) + float(a[0]) + float(b[0])
    if comparator in ("dot", "cos"):
        return float(a @ b)
    if comparator == "l2":
        d = a - b
        return -math.sqrt(max(float(d @ d), 1e-30))
    if comparator == "squared_l2":  # model.py:300-303
        d = a - b
        return -float(d @ d)
    raise NotImplementedError(comparator)


def scores(cfg, w_lhs, w_rhs, lhs, rhs, rel, uniform_lhs, uniform_rhs, lhs_op, rhs_op):
    """Returns (lhs_pos[B], rhs_pos[B], lhs_neg[B,Nl], rhs_neg[B,Nr]) in
    float64.  Arguments are numpy arrays; ``rel`` is an int or an int array."""
    w_lhs = np.asarray(w_lhs, dtype=np.float64)
    w_rhs = np.asarray(w_rhs, dtype=np.float64)
    lhs_op = {k: np.asarray(v, dtype=np.float64) for k, v in (lhs_op or {}).items()} or None
    rhs_op = {k: np.asarray(v, dtype=np.float64) for k, v in (rhs_op or {}).items()} or None
    num_pos = len(lhs)
    chunk, _, mode = cfg.chunking(num_pos)
    n_batch = chunk if mode == "batch_uniform" else 0
    n_uni = cfg.num_uniform_negs
    n_l = 0 if cfg.disable_lhs_negs else n_batch + n_uni
    n_r = 0 if cfg.disable_rhs_negs else n_batch + n_uni
    if mode == "all":  # every entity of the side's type, the edge's own entity masked (model.py:582-618)
        n_l = 0 if cfg.disable_lhs_negs else len(w_lhs)
        n_r = 0 if cfg.disable_rhs_negs else len(w_rhs)
    lpos = np.zeros(num_pos)
    rpos = np.zeros(num_pos)
    lneg = np.zeros((num_pos, n_l))
    rneg = np.zeros((num_pos, n_r))
    cmp_ = cfg.comparator
    bias = bool(getattr(cfg, "bias", False))
    name = cfg.operator
    for e in range(num_pos):
        c, i = divmod(e, chunk)
        r = int(rel) if np.ndim(rel) == 0 else int(rel[e])
        u_raw, v_raw = w_lhs[lhs[e]], w_rhs[rhs[e]]
        if not cfg.dynamic:
            a_for_rneg = _prep(cmp_, u_raw, bias)                      # f(u)
            a_for_lneg = _prep(cmp_, _op(name, v_raw, rhs_op, r), bias)  # f(op_r(v))
            lpos[e] = rpos[e] = _kappa(cmp_, a_for_rneg, a_for_lneg, bias)
        else:
            a_for_lneg = _prep(cmp_, _op(name, v_raw, rhs_op, r), bias)  # f(op^rhs_r(v))
            a_for_rneg = _prep(cmp_, _op(name, u_raw, lhs_op, r), bias)  # f(op^lhs_r(u))
            lpos[e] = _kappa(cmp_, _prep(cmp_, u_raw, bias), a_for_lneg, bias)
            rpos[e] = _kappa(cmp_, _prep(cmp_, v_raw, bias), a_for_rneg, bias)
        for side, n_cols, out, a_vec in (("l", n_l, lneg, a_for_lneg), ("r", n_r, rneg, a_for_rneg)):
            if n_cols == 0:
                continue
            ids = lhs if side == "l" else rhs
            table = w_lhs if side == "l" else w_rhs
            uni = uniform_lhs if side == "l" else uniform_rhs
            neg_op = rhs_op if (side == "r" and not cfg.dynamic) else None
            for j in range(n_batch):
                other = c * chunk + j
                if other >= num_pos or j == i:
                    out[e, j] = -1e9
                    continue
                b_vec = _prep(cmp_, _op(name, table[ids[other]], neg_op, r), bias)
                out[e, j] = _kappa(cmp_, a_vec, b_vec, bias)
            if mode == "all":
                for j in range(n_cols):
                    if j == ids[e]:
                        out[e, j] = -1e9
                        continue
                    out[e, j] = _kappa(cmp_, a_vec, _prep(cmp_, _op(name, table[j], neg_op, r), bias), bias)
                continue
            for j in range(n_uni):
                b_vec = _prep(cmp_, _op(name, table[uni[c][j]], neg_op, r), bias)
                out[e, n_batch + j] = _kappa(cmp_, a_vec, b_vec, bias)
    return lpos, rpos, lneg, rneg


def loss(name: str, pos: np.ndarray, neg: np.ndarray, margin: float) -> float:
    """Textbook forms of the three losses (docs/source/loss_optimization.rst;
    the softmax keeps the positive in the partition function as
    losses.py:143-159 does)."""
    total = 0.0
    n = neg.shape[1]
    for i in range(len(pos)):
        if name == "ranking":
            for j in range(n):
                total += max(0.0, margin - pos[i] + neg[i, j])
        elif name == "logistic":
            total += math.log1p(math.exp(-abs(pos[i]))) + max(-pos[i], 0.0)
            for j in range(n):
                t = neg[i, j]
                total += (math.log1p(math.exp(-abs(t))) + max(t, 0.0)) / n
        elif name == "softmax":
            if n == 0:
                continue
            m = max(pos[i], neg[i].max())
            z = math.exp(pos[i] - m) + sum(math.exp(t - m) for t in neg[i])
            total += -pos[i] + m + math.log(z)
        else:
            raise NotImplementedError(name)
    return total

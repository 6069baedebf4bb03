"""Helpers shared by the GPU parity tests: power-law ids, a float64 copy of an
oracle state, the float64-anchored comparison and the hinge-tie census."""
import copy
import math

import torch


def zipf_ids(n, num, s, gen):
    """ids in [0, num) with P(rank r) ~ r^-s, ranks mapped through a fixed stride permutation."""
    u = torch.rand(n, generator=gen, dtype=torch.float64)
    if abs(s - 1.0) < 1e-9:
        r = torch.exp(u * math.log(num))
    else:
        a = 1.0 - s
        r = ((num ** a - 1.0) * u + 1.0) ** (1.0 / a)
    ranks = (r.floor().long() - 1).clamp_(0, num - 1)
    return (ranks * 7919 + 13) % num  # 7919 is prime: a bijection unless it divides num


def double_state(st):
    """A float64 copy of an oracle TrainState (tables shared where `st` shares them)."""
    st64 = copy.deepcopy(st)
    for name in ("w_lhs", "g_lhs", "w_rhs", "g_rhs"):
        setattr(st64, name, getattr(st64, name).double())
    if st.shared:
        st64.w_rhs, st64.g_rhs = st64.w_lhs, st64.g_lhs
    for dct in (st64.lhs_op, st64.rhs_op, st64.lhs_op_sum, st64.rhs_op_sum):
        for k in dct:
            dct[k] = dct[k].double()
    if st.glob_lhs is not None:
        one = st.glob_rhs is st.glob_lhs
        st64.glob_lhs, st64.glob_lhs_sum = st64.glob_lhs.double(), st64.glob_lhs_sum.double()
        if one:
            st64.glob_rhs, st64.glob_rhs_sum = st64.glob_lhs, st64.glob_lhs_sum
        else:
            st64.glob_rhs, st64.glob_rhs_sum = st64.glob_rhs.double(), st64.glob_rhs_sum.double()
    return st64


class Census:
    """Counts, over one test, how many entries passed on the plain criterion and
    how many needed the float64 anchor."""

    def __init__(self):
        self.entries = 0
        self.anchored = 0

    def __str__(self):
        return f"{self.entries} entries, {self.anchored} passed on the float64 anchor only"


def anchored_close(got, ref32, exact, rtol, what, census=None, loose=None, loose_bound=0.0, slack=None):
    """The stated criterion first: `got` within rtol (relative, with a floor of
    rtol/10 of the tensor's largest entry) of the CPU path's fp32 result `ref32`.
    An entry that misses it must be explained by fp32 rounding alone: it lies
    within rtol of the float64 evaluation `exact`, or no further from it than three
    times the largest distance the CPU path's own fp32 result has from `exact` in
    the same row (per tensor for vectors).  A row that many edges of a power-law
    batch name sums thousands of gradient rows, and `l2` cancels ||a||^2 - 2ab +
    ||b||^2: their fp32 results depend on the order of summation by more than rtol
    in the reference as much as here.  `loose` marks entries held to `loose_bound`
    (absolute) instead; `slack` is an absolute allowance per entry on top of both
    criteria (adagrad_noise_slack)."""
    got = got.detach().cpu().double()
    ref = ref32.detach().double()
    exact = exact.detach().double()
    assert got.shape == ref.shape == exact.shape, (what, got.shape, ref.shape, exact.shape)
    if got.numel() == 0:
        return
    scale = max(ref.abs().max().item(), 1e-30)
    floor = 0.1 * rtol * scale
    if slack is not None:
        floor = floor + slack.double()
    plain = (got - ref).abs() <= rtol * ref.abs() + floor
    noise = (ref - exact).abs()
    noise = noise.amax(dim=-1, keepdim=True) if noise.dim() >= 2 else noise.max()
    err = (got - exact).abs()
    anchored = err <= rtol * exact.abs() + floor + 3.0 * noise
    ok = plain | anchored
    if loose is not None:
        ok = torch.where(loose, err <= loose_bound, ok)
    if census is not None:
        census.entries += got.numel()
        census.anchored += int((~plain & ok).sum())
    bad = ~ok
    assert not bad.any(), (what, "max err vs fp32", (got - ref).abs().max().item(), "vs float64", err.max().item(),
                           "scale", scale, "count", int(bad.sum()), "fp32 reference noise", float(noise.max()))


def adagrad_noise_slack(grads, lr, rel_noise=2e-7):
    """How far fp32 rounding of the gradients alone can move a parameter over a
    sequence of AsyncAdagrad steps (async_adagrad.py:75-85).  `grads`: the exact
    gradient of each step, in order, leading axis = relation.  A gradient entry is a
    cancelling sum over a batch; in fp32 it carries an absolute error of about
    rel_noise times the largest entry of its relation's slice, whatever its own
    size.  Step k moves an entry by lr * g_k / sqrt(sum_{j<=k} g_j^2), so that error
    moves it by up to lr * error / sqrt(sum): negligible where the gradients are of
    ordinary size, a visible fraction of lr where an entry's gradients so far are
    all tiny (and never more than 2 lr, a flipped sign)."""
    total = torch.zeros_like(grads[0], dtype=torch.float64)
    slack = torch.zeros_like(total)
    for g in grads:
        g = g.double()
        total = total + g * g
        err = rel_noise * g.abs().reshape(g.shape[0], -1).amax(dim=1).reshape(-1, *([1] * (g.dim() - 1)))
        step = torch.where(total > 0, lr * err / total.sqrt().clamp_min(1e-300), torch.zeros_like(total))
        slack = slack + step.clamp_max(2 * lr)
    return slack


def anchored_state(cfg, runner, st, st64, rtol, tag, census=None, loose_rows=None, loose_steps=0, param_slack=None):
    """Tables, Adagrad sums, operator parameters and global embeddings of a
    StepRunner against the oracle's fp32 and float64 states.  `loose_rows` =
    (bool[rows of lhs table], bool[rows of rhs table]): rows a hinge tie reaches;
    they, and every operator parameter, may then differ by `loose_steps` Adagrad
    steps (a step never exceeds the step size); their Adagrad sums are not compared.
    `param_slack` = {"rhs_op" | "lhs_op": {name: adagrad_noise_slack(...)}}."""
    rel_lr = cfg.relation_lr if cfg.relation_lr is not None else cfg.lr
    inf = float("inf")

    def rows(side, like, bound):
        if loose_rows is None:
            return {}
        m = loose_rows[side]
        return dict(loose=m.unsqueeze(1).expand_as(like) if like.dim() == 2 else m, loose_bound=bound)

    anchored_close(runner.w_lhs, st.w_lhs, st64.w_lhs, rtol, tag + " w_lhs", census, **rows(0, st.w_lhs, loose_steps * cfg.lr))
    anchored_close(runner.g_lhs, st.g_lhs, st64.g_lhs, rtol, tag + " g_lhs", census, **rows(0, st.g_lhs, inf))
    if not st.shared:
        anchored_close(runner.w_rhs, st.w_rhs, st64.w_rhs, rtol, tag + " w_rhs", census, **rows(1, st.w_rhs, loose_steps * cfg.lr))
        anchored_close(runner.g_rhs, st.g_rhs, st64.g_rhs, rtol, tag + " g_rhs", census, **rows(1, st.g_rhs, inf))

    def params(like, bound, slack=None):
        if loose_rows is None:
            return dict(slack=slack)
        return dict(loose=torch.ones_like(like, dtype=torch.bool), loose_bound=bound)

    for name in ("rhs_op", "rhs_op_sum", "lhs_op", "lhs_op_sum"):
        got, want, exact = getattr(runner, name), getattr(st, name), getattr(st64, name)
        for k in want:
            slack = (param_slack or {}).get(name, {}).get(k)
            anchored_close(got[k], want[k], exact[k], rtol, f"{tag} {name}.{k}", census,
                           **params(want[k], inf if name.endswith("sum") else loose_steps * rel_lr, slack))
    if st.glob_lhs is not None:
        for i, (w, w64, s, s64) in enumerate(((st.glob_lhs, st64.glob_lhs, st.glob_lhs_sum, st64.glob_lhs_sum),
                                              (st.glob_rhs, st64.glob_rhs, st.glob_rhs_sum, st64.glob_rhs_sum))):
            anchored_close(runner.global_embs[i], w, w64, rtol, f"{tag} global {i}", census, **params(w, loose_steps * rel_lr))
            anchored_close(runner.global_sums[i], s, s64, rtol, f"{tag} global sum {i}", census, **params(s, inf))


def hinge_ties(cfg, scores, eps=2e-6):
    """Number of negatives whose hinge argument (neg - pos) + margin lies within
    eps of 0: max(0, x) has a gradient of 0 on one side and 1 on the other, so two
    correct fp32 evaluations may take different sides there."""
    n = 0
    for pos, neg in ((scores.lhs_pos, scores.lhs_neg), (scores.rhs_pos, scores.rhs_neg)):
        x = (neg - pos.unsqueeze(1)) + cfg.margin
        n += int((x.abs() < eps).sum())
    return n


def tie_free_batches(cfg, st64, candidates, steps, eps):
    """The first `steps` of `candidates` that, taken in order along a float64 run of
    the oracle from `st64`, have no live hinge argument (neg - pos) + margin within
    eps * max(1, largest |score|) of 0; a candidate that has one is skipped.  `st64`
    is advanced through the kept batches.  Returns (kept, number of candidates looked at)."""
    from oracle import step as ostep

    kept, looked = [], 0
    for b in candidates:
        if len(kept) == steps:
            break
        looked += 1
        sc = ostep.forward_backward(cfg, st64, *b, keep_scores=True)[0].scores
        nearest, largest = float("inf"), 1.0
        for pos, neg in ((sc.lhs_pos, sc.lhs_neg), (sc.rhs_pos, sc.rhs_neg)):
            live = neg > -1e8  # masked entries hold -1e9 and never reach the hinge
            x = ((neg - pos.unsqueeze(1)) + cfg.margin)[live]
            if x.numel():
                nearest = min(nearest, float(x.abs().min()))
                largest = max(largest, float(neg[live].abs().max()), float(pos.abs().max()))
        if nearest < eps * largest:
            continue
        ostep.train_step(cfg, st64, *b)
        kept.append(b)
    return kept, looked


def hinge_tie_rows(cfg, scores, lhs, rhs, uniform_lhs, uniform_rhs, eps=2e-6):
    """(rows of the lhs table, rows of the rhs table) that a hinge tie of this batch
    reaches: the tied edge's two entities and the tied negative's entity (a batch
    negative is another edge of the chunk, model.py:547; a uniform one is named by
    the index arrays)."""
    chunk, _, _ = cfg.chunking(lhs.shape[0])
    has_batch_negs = cfg.num_batch_negs > 0
    out = ([], [])
    for side, pos, neg, ids, uniform in ((0, scores.lhs_pos, scores.lhs_neg, lhs, uniform_lhs),
                                         (1, scores.rhs_pos, scores.rhs_neg, rhs, uniform_rhs)):
        x = (neg - pos.unsqueeze(1)) + cfg.margin
        for i, j in (x.abs() < eps).nonzero().tolist():
            out[0].append(int(lhs[i]))
            out[1].append(int(rhs[i]))
            c = i // chunk
            if has_batch_negs and j < chunk:
                out[side].append(int(ids[c * chunk + j]))
            else:
                out[side].append(int(uniform[c, j - (chunk if has_batch_negs else 0)]))
    return out


def violator_ties(pos, neg):
    """Negatives whose score equals the positive's up to fp32 rounding of a score
    (about 1e-6 of the largest score of the batch): `neg > pos` may fall either way."""
    p = pos.unsqueeze(1)
    window = 2e-5 * p.abs() + 2e-6 * max(float(neg.abs().max()) if neg.numel() else 0.0, float(pos.abs().max()))
    return int(((neg - p).abs() <= window).sum())

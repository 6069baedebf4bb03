"""The BASELINE configurations at their full shapes (table sizes, batch size,
negatives, dim), through the C ABI.

The training step only touches the rows a batch names, so the CPU oracle runs
on a compacted copy of those rows (ids renumbered by torch.unique) while the
GPU works on the full table: that covers 64-bit addressing (the dim-1024 table
holds 4.96e9 floats), power-law duplicates and the real workspace sizes, and
the rest of the table must come back bit-identical.  The permutation helpers
are checked through size-independent properties (round trips, conservation)."""
import copy
import math

import pytest
import torch

from oracle import step as ostep
from test_gpu_step import say

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


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


def close_to_exact(got, ref32, exact, rtol, what, loose=None, loose_bound=0.0):
    """`got` lies within rtol of the float64 evaluation, or within three times the
    distance the reference's own fp32 evaluation (`ref32`) lies from it.  A row
    that half of a power-law batch names sums thousands of gradient rows, and an
    operator-parameter gradient sums a whole batch with cancellation: their fp32
    results depend on the order of summation by more than 1e-5, in the reference
    as much as here.  The noise allowance is the largest deviation of `ref32` in
    the same row (per tensor for vectors)."""
    got = got.detach().cpu().double()
    exact = exact.detach().double()
    noise = (ref32.detach().double() - exact).abs()
    noise = noise.amax(dim=-1, keepdim=True) if noise.dim() >= 2 else noise.max()
    scale = max(exact.abs().max().item(), 1e-30)
    err = (got - exact).abs()
    bound = rtol * exact.abs() + 1e-6 * scale * rtol / 1e-5 + 3.0 * noise
    if loose is not None:
        bound = torch.where(loose, torch.full_like(bound, loose_bound), bound)
    bad = err > bound
    assert not bad.any(), (what, "max err", err.max().item(), "scale", scale, "count", int(bad.sum()),
                           "fp32 reference noise", noise.max().item())


FULL = {
    # name: entities, relations, dim, B, batch negs, uniform negs, operator, comparator, loss, dynamic, zipf, two tables
    "cfg1": dict(entities=100_000, relations=1, dim=100, batch=1000, nb=50, nu=50, operator="none", comparator="dot",
                 loss="ranking", dynamic=False, zipf=None, two_tables=False),
    "cfg2-standard": dict(entities=14_951, relations=1345, dim=400, batch=1000, nb=50, nu=1000,
                          operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, zipf=1.1,
                          two_tables=False),
    # ... with the N3 regularizer of the reference's FB15k example (fb15k_config_cpu.py:41)
    "cfg2-standard-n3": dict(entities=14_951, relations=1345, dim=400, batch=1000, nb=50, nu=1000,
                             operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False, zipf=1.1,
                             two_tables=False, reg=1e-3),
    "cfg2-dynamic": dict(entities=14_951, relations=1345, dim=400, batch=1000, nb=50, nu=1000,
                         operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=True, zipf=1.1,
                         two_tables=False),
    "cfg2-1000-batch-negs": dict(entities=14_951, relations=1345, dim=400, batch=1000, nb=1000, nu=0,
                                 operator="complex_diagonal", comparator="dot", loss="softmax", dynamic=False,
                                 zipf=1.1, two_tables=False),
    # the graph as BASELINE states it: out-degree Zipf(2.0) capped at 20 000, targets by preferential attachment
    # (bench.livejournal_like_edges, all 68 993 773 edges, the same generator the bench line runs on)
    "cfg3": dict(entities=4_847_571, relations=1, dim=1024, batch=10_000, nb=1000, nu=100, operator="none",
                 comparator="dot", loss="softmax", dynamic=False, zipf=2.0, two_tables=False, graph="livejournal"),
    # a harsher graph than stated: both endpoints i.i.d. Zipf(2.0) without a cap, one entity holds 60 % of a batch
    "cfg3-hot": dict(entities=4_847_571, relations=1, dim=1024, batch=10_000, nb=1000, nu=100, operator="none",
                     comparator="dot", loss="softmax", dynamic=False, zipf=2.0, two_tables=False),
    "cfg4": dict(entities=10_413_058, relations=1, dim=100, batch=1000, nb=50, nu=50, operator="translation",
                 comparator="l2", loss="ranking", dynamic=False, zipf=1.8, two_tables=True),
    "cfg5-standard": dict(entities=2_000_000, relations=500, dim=256, batch=2000, nb=100, nu=100, operator="linear",
                          comparator="cos", loss="logistic", dynamic=False, zipf=None, two_tables=False),
    "cfg5-dynamic": dict(entities=2_000_000, relations=500, dim=256, batch=2000, nb=100, nu=100, operator="linear",
                         comparator="cos", loss="logistic", dynamic=True, zipf=None, two_tables=False),
}


@pytest.mark.parametrize("name", sorted(FULL))
@pytest.mark.parametrize("workers", [1, 2])
def test_full_shape_step(pbg, name, workers):
    say("full shape", name, workers)
    w = FULL[name]
    e, d, b, r = w["entities"], w["dim"], w["batch"], w["relations"]
    cfg = ostep.StepConfig(dim=d, operator=w["operator"], comparator=w["comparator"], loss=w["loss"], margin=0.1,
                           num_batch_negs=w["nb"], num_uniform_negs=w["nu"], dynamic=w["dynamic"], num_relations=r,
                           lr=0.1, relation_lr=0.01, relation_weights=[1.0] * r,
                           regularization_coef=w.get("reg", 0.0))
    _, c, _ = cfg.chunking(b)
    u = w["nu"]
    gen = torch.Generator().manual_seed(7)
    dgen = torch.Generator(device=DEV).manual_seed(7)
    # N(0, 1e-3) as the workloads are specified, except where operator parameters are
    # trained: their gradients would be ~1e-10, the size of Adagrad's epsilon, where
    # lr * g / (|g| + 1e-10) turns fp32 rounding noise in g into 1e-6 parameter noise
    scale = 1e-3 if w["operator"] == "none" else (0.1 if w["comparator"] == "dot" else 0.3)
    tables = [torch.randn(e, d, generator=dgen, device=DEV) * scale]
    if w["two_tables"]:
        tables.append(torch.randn(e, d, generator=dgen, device=DEV) * scale)
    before = [t.clone() for t in tables]
    sums = [torch.zeros(e, device=DEV) for _ in tables]

    def draw(n):
        return zipf_ids(n, e, w["zipf"], gen) if w["zipf"] else torch.randint(0, e, (n,), generator=gen)

    graph = None
    if w.get("graph") == "livejournal":
        import bench
        graph = bench.livejournal_like_edges(e, 68_993_773, w["zipf"], 20_000, dgen, DEV)
        graph = (graph[0][:workers * b].cpu(), graph[1][:workers * b].cpu())
        torch.cuda.empty_cache()

    batches = []
    for k in range(workers):
        lhs, rhs = (graph[0][k * b:(k + 1) * b], graph[1][k * b:(k + 1) * b]) if graph else (draw(b), draw(b))
        ul = torch.randint(0, e, (c, u), generator=gen)
        ur = torch.randint(0, e, (c, u), generator=gen)
        if w["dynamic"]:
            rel = zipf_ids(b, r, 1.2, gen).sort().values  # mixed batch sorted by relation
        else:
            rel = int(torch.randint(0, r, (1,), generator=gen))
        batches.append((lhs, rhs, rel, ul, ur))

    # compacted tables for the oracle
    def side_ids(side):
        return torch.cat([torch.cat([bt[side], bt[3 + side].reshape(-1)]) for bt in batches])

    if w["two_tables"]:
        uniq = [torch.unique(side_ids(0)), torch.unique(side_ids(1))]
    else:
        uniq = [torch.unique(torch.cat([side_ids(0), side_ids(1)]))]
    small = [tables[i][uniq[i].to(DEV)].cpu() for i in range(len(tables))]
    st = ostep.make_state(cfg, small[0], small[1] if w["two_tables"] else None)
    for dct in (st.lhs_op, st.rhs_op):
        for k in dct:
            dct[k] = dct[k] + 0.1 * torch.randn(dct[k].shape, generator=gen)

    # The same state in float64: "exact" arithmetic, against which the rounding
    # noise of the reference's own fp32 evaluation is measured row by row.
    st64 = copy.deepcopy(st)
    for name in ("w_lhs", "g_lhs", "w_rhs", "g_rhs"):
        setattr(st64, name, getattr(st64, name).double())
    if not w["two_tables"]:
        st64.w_rhs, st64.g_rhs = st64.w_lhs, st64.g_lhs
    for dct in (st64.lhs_op, st64.rhs_op, st64.lhs_op_sum, st64.rhs_op_sum):
        for k in dct:
            dct[k] = dct[k].double()

    def remap(ids, table):
        return torch.searchsorted(uniq[table], ids)

    t_r = 1 if w["two_tables"] else 0
    small_batches = [(remap(bt[0], 0), remap(bt[1], t_r), bt[2], remap(bt[3], 0), remap(bt[4], t_r)) for bt in batches]

    spec = pbg.StepSpec(dim=d, batch_size=b, num_workers=workers, num_batch_negs=w["nb"], num_uniform_negs=u,
                        operator=w["operator"], dynamic=w["dynamic"], num_relations=r, comparator=w["comparator"],
                        loss=w["loss"], margin=0.1, lr=0.1, relation_lr=0.01, regularization_coef=w.get("reg", 0.0))
    ops = [{k: v.clone().to(DEV) for k, v in dct.items()} for dct in (st.rhs_op, st.rhs_op_sum, st.lhs_op, st.lhs_op_sum)]
    runner = pbg.StepRunner(spec, tables[0], sums[0], tables[1] if w["two_tables"] else None,
                            sums[1] if w["two_tables"] else None, ops[0], ops[1], ops[2], ops[3])
    lhs = torch.stack([bt[0] for bt in batches]).to(DEV)
    rhs = torch.stack([bt[1] for bt in batches]).to(DEV)
    if w["dynamic"]:
        rel = torch.stack([bt[2] for bt in batches]).to(DEV)
    else:
        rel = torch.tensor([bt[2] for bt in batches], dtype=torch.int64, device=DEV)
    ul = torch.stack([bt[3] for bt in batches]).contiguous().to(DEV) if u else None
    ur = torch.stack([bt[4] for bt in batches]).contiguous().to(DEV) if u else None
    runner.train(lhs, rhs, rel, ul, ur)
    torch.cuda.synchronize()

    outs = ostep.train_lockstep(cfg, st, small_batches)
    # Exact operator-parameter gradients of every batch (all batches read the state
    # as it is on entry).  Where |g| is within a factor 1e4 of Adagrad's epsilon,
    # p -= lr * g / (sqrt(sum) + 1e-10) amplifies fp32 rounding noise in g (about
    # 1e-7 of its terms) to a visible fraction of a step; a step never exceeds lr.
    tiny = {"lhs_op": {}, "rhs_op": {}}
    for bt in small_batches:
        _, grads = ostep.forward_backward(cfg, st64, *bt)
        for nm, gd in (("lhs_op", grads.lhs_op), ("rhs_op", grads.rhs_op)):
            for k, gv in gd.items():
                t = gv.abs() < 1e-6
                tiny[nm][k] = t | tiny[nm][k] if k in tiny[nm] else t
    ostep.train_lockstep(cfg, st64, small_batches)
    rtol = 1e-5
    for k, out in enumerate(outs):
        assert float(runner.loss_out[k]) == pytest.approx(out.loss, rel=rtol, abs=1e-6), ("loss", k)
        assert float(runner.reg_out[k]) == pytest.approx(out.reg, rel=1e-5), ("reg", k)
    want_w = [(st.w_lhs, st64.w_lhs)] + ([(st.w_rhs, st64.w_rhs)] if w["two_tables"] else [])
    want_g = [(st.g_lhs, st64.g_lhs)] + ([(st.g_rhs, st64.g_rhs)] if w["two_tables"] else [])
    for i in range(len(tables)):
        ids = uniq[i].to(DEV)
        close_to_exact(tables[i][ids], *want_w[i], rtol, f"table {i}")
        close_to_exact(sums[i][ids], *want_g[i], rtol, f"adagrad sum {i}")
        # every other row comes back bit-identical, its Adagrad sum still zero
        changed = (tables[i] != before[i]).any(dim=1)
        changed[ids] = False
        assert not bool(changed.any()), f"table {i}: rows outside the batch changed"
        touched = sums[i] != 0
        touched[ids] = False
        assert not bool(touched.any()), f"adagrad sum {i}: rows outside the batch changed"
    for nm, got, want, exact in (("rhs_op", ops[0], st.rhs_op, st64.rhs_op),
                                 ("rhs_op_sum", ops[1], st.rhs_op_sum, st64.rhs_op_sum),
                                 ("lhs_op", ops[2], st.lhs_op, st64.lhs_op),
                                 ("lhs_op_sum", ops[3], st.lhs_op_sum, st64.lhs_op_sum)):
        for k in want:
            loose = tiny[nm][k] if nm in tiny else None
            close_to_exact(got[k], want[k], exact[k], rtol, f"{nm}.{k}", loose, workers * 0.01 * 1.01)


def test_gather_full_tables_bit_exact(pbg):
    """A gather through a permutation followed by a gather through its inverse
    returns the table; checked on the dim-100 partition of cfg4 (10.4M rows) and
    on 2M rows of the dim-1024 table of cfg3 (8 GB)."""
    from pytorch_biggraph_amd import native

    gen = torch.Generator(device=DEV).manual_seed(3)
    for rows, dim in ((10_413_058, 100), (2_000_000, 1024)):
        say("gather", rows, dim)
        table = torch.randn(rows, dim, generator=gen, device=DEV)
        perm = torch.randperm(rows, generator=gen, device=DEV)
        inv = native.reverse_permutation(perm)
        moved = native.gather_rows(table, perm)
        assert torch.equal(moved[12345], table[perm[12345]])
        back = native.gather_rows(moved, inv)
        assert torch.equal(back, table)
        del table, moved, back


def test_permutation_helpers_at_cfg4_size(pbg):
    """randperm / reverse_permutation / shuffle on the 41.65M entities of cfg4."""
    from pytorch_biggraph_amd import native

    n = 41_652_230
    say("permutation helpers", n)
    perm = native.randperm(n, 5, DEV)
    assert int(perm.min()) == 0 and int(perm.max()) == n - 1
    assert torch.equal(torch.sort(perm).values, torch.arange(n, device=DEV))
    rev = native.reverse_permutation(perm)
    assert torch.equal(rev[perm], torch.arange(n, device=DEV))
    part = 10_413_058
    sub = native.randperm(part, 6, DEV)
    rows = torch.randn(part, 100, device=DEV)
    keep = rows.clone()
    native.shuffle_rows(rows, sub)                               # rows[sub[i]] <- rows[i]
    assert torch.equal(rows[sub[:1000]], keep[:1000])
    native.shuffle_rows(rows, native.reverse_permutation(sub))   # and back (train_gpu.py:627-632)
    assert torch.equal(rows, keep)


def test_sub_bucket_at_bucket_size(pbg):
    """One bucket of cfg4 (91.8M edges) split 8 x 8: every edge lands in the
    sub-bucket its permuted ids name, offsets add up, and the order inside a
    sub-bucket is the input order."""
    from pytorch_biggraph_amd import native

    n, ents, parts = 91_772_824, 10_413_058, 8
    say("sub_bucket", n)
    gen = torch.Generator(device=DEV).manual_seed(11)
    lhs = torch.randint(0, ents, (n,), generator=gen, device=DEV)
    rhs = torch.randint(0, ents, (n,), generator=gen, device=DEV)
    rel = torch.zeros(n, dtype=torch.int64, device=DEV)
    lp = native.randperm(ents, 1, DEV)
    rp = native.randperm(ents, 2, DEV)
    size = (ents + parts - 1) // parts
    lo, ro, relo = torch.empty_like(lhs), torch.empty_like(rhs), torch.empty_like(rel)
    offsets = native.sub_bucket(lhs, rhs, rel, [lp], [rp], [size], [size], parts, parts, False, lo, ro, relo).cpu()
    assert int(offsets[0]) == 0 and int(offsets[-1]) == n
    code = (lp[lhs] // size) * parts + rp[rhs] // size
    counts = torch.bincount(code, minlength=parts * parts).cpu()
    assert torch.equal(offsets[1:] - offsets[:-1], counts)
    for i, j in ((0, 0), (3, 5), (7, 7)):
        sel = code == i * parts + j
        a, b = int(offsets[i * parts + j]), int(offsets[i * parts + j + 1])
        assert torch.equal(lo[a:b], lp[lhs[sel]] % size) and torch.equal(ro[a:b], rp[rhs[sel]] % size), (i, j)
    assert int(relo.abs().max()) == 0

#!/usr/bin/env python3
"""Throughput of the PBG training step on one MI355X.

    python bench.py [--gpus 1] [--steps N] [--warmup W] [--workload NAME] [--workers 64]

A "step" is one call of pbg_train_step: `workers` batches of `batch_size` edges
through the whole hot path (gather, operator, scoring against batch + uniform
negatives, loss, backward, RowAdagrad and operator Adagrad), processed like
`workers` HOGWILD processes in lock-step (all read, then all write in order).
`--steps` and `--warmup` count calls and never change `workers`; `--workers 1` is
the strictly sequential single-process order.  Before the warm-up calls the device
is kept busy for `--preheat-ms` (200) with the same calls on a scratch copy of the
state, so that a short run is not timed while the clocks still settle.  Prints ONE
JSON line.

Without `--workload` the line is cfg1's (the configuration the metric is quoted
on) and carries, under "configs", the same measurement for every other BASELINE
configuration (cfg2 standard and with one relation per edge, cfg2b = cfg2 with
1000 batch negatives, cfg2cos = cfg2's shape under the reference's default
comparator, cfg3 on the graph BASELINE states and on the harsher cfg3-hot, cfg4,
cfg5), each with its own roofline entry, strictly sequential
value and CPU baseline; under "k_sweep" cfg1 at 1 ... 64 batches per call; under
"standalone" the gather / RowAdagrad kernels alone; under "perm_kernels" the
permutation helpers; under "cfg4_epoch" one pass over cfg4's 16 buckets with
partition swaps.  All CPU legs run first, before the process opens the GPU.
`--workload NAME` measures that one workload only (`--extras` adds the rest).
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FP32_MFMA_PEAK_TFLOPS = 157.3
FP16_MFMA_PEAK_TFLOPS = 2500.0  # dense fp16, what --half-precision's products are priced against
# HBM bytes per launch of (workload, kernel, workers), from the rocprofv3 FETCH_SIZE /
# WRITE_SIZE runs summarised in profiles/train_step_pmc_traffic.md (not measured live);
# any other combination reports null.
TRAFFIC = {("cfg1", "fused_chunk", 64): 233.3e6, ("cfg4", "fused_chunk", 64): 225.5e6,
           ("cfg2", "stream_chunk", 64): 13957.7e6}

# name -> the fields of BASELINE.json's configs.  `graph` says how the edge list is drawn:
#   (none)       both endpoints uniform, or with `zipf` both i.i.d. P(rank r) ~ r^-zipf over shuffled ids (no cap)
#   livejournal  out-degrees P(k) ~ k^-zipf on 2 <= k <= degree_cap, targets by preferential attachment
WORKLOADS = {
    "cfg1": dict(desc="single relation, identity/dot/ranking(0.1), dim 100, 100k entities, B=1000, 50 batch + 50 uniform negatives",
                 entities=100_000, edges=1_000_000, dim=100, batch=1000, batch_negs=50, uniform_negs=50,
                 operator="none", comparator="dot", loss="ranking", relations=1, dynamic=False,
                 init_scale=1e-3, zipf=None, two_tables=False),
    "cfg2": dict(desc="1345 relations, complex_diagonal/dot/softmax, dim 400, 14951 entities, B=1000, chunk 50 + 1000 uniform negatives, single-relation batches",
                 entities=14_951, edges=483_142, dim=400, batch=1000, batch_negs=50, uniform_negs=1000,
                 operator="complex_diagonal", comparator="dot", loss="softmax", relations=1345, dynamic=False,
                 init_scale=1e-3, zipf=1.1, two_tables=False),
    "cfg2b": dict(desc="cfg2 read as 1000 batch negatives (one chunk of 1000, no uniform negatives): 1345 relations, complex_diagonal/dot/softmax, dim 400, 14951 entities, B=1000, single-relation batches",
                  entities=14_951, edges=483_142, dim=400, batch=1000, batch_negs=1000, uniform_negs=0,
                  operator="complex_diagonal", comparator="dot", loss="softmax", relations=1345, dynamic=False,
                  init_scale=1e-3, zipf=1.1, two_tables=False),
    "cfg3": dict(desc="single relation, identity/dot/softmax, dim 1024, 4,847,571 entities, B=10000, 1000 batch + 100 uniform negatives; "
                      "graph: all 68,993,773 edges drawn, out-degree P(k) ~ k^-2 on 2..20000 (capped), targets by preferential attachment "
                      "(Barabasi-Albert: P(v) ~ in-degree + mean out-degree among the entities arrived so far), edge order shuffled",
                 entities=4_847_571, edges=68_993_773, dim=1024, batch=10_000, batch_negs=1000, uniform_negs=100,
                 operator="none", comparator="dot", loss="softmax", relations=1, dynamic=False,
                 init_scale=1e-3, zipf=2.0, graph="livejournal", degree_cap=20_000, two_tables=False),
    "cfg3-hot": dict(desc="cfg3's shape on a harsher graph than BASELINE states (a stress case for the update stage): both endpoints "
                          "i.i.d. Zipf(2.0) over the 4,847,571 entities with NO degree cap, so one entity holds about 60% of every batch",
                     entities=4_847_571, edges=4_000_000, dim=1024, batch=10_000, batch_negs=1000, uniform_negs=100,
                     operator="none", comparator="dot", loss="softmax", relations=1, dynamic=False,
                     init_scale=1e-3, zipf=2.0, two_tables=False),
    "cfg4": dict(desc="one bucket of 4x4: translation/l2/ranking, dim 100, two resident partitions of 10.4M entities, B=1000, 50 + 50 negatives, both endpoints Zipf(1.8)",
                 entities=10_413_058, edges=4_000_000, dim=100, batch=1000, batch_negs=50, uniform_negs=50,
                 operator="translation", comparator="l2", loss="ranking", relations=1, dynamic=False,
                 init_scale=1e-3, zipf=1.8, two_tables=True),
    "cfg5": dict(desc="500 relations (dynamic: one per edge), linear/cos/logistic, dim 256, 2M entities, B=2000, 100 batch + 100 uniform negatives, mixed batches sorted by relation, relation ids Zipf(1.2)",
                 entities=2_000_000, edges=4_000_000, dim=256, batch=2000, batch_negs=100, uniform_negs=100,
                 operator="linear", comparator="cos", loss="logistic", relations=500, dynamic=True,
                 init_scale=1e-3, zipf=None, rel_zipf=1.2, two_tables=False),
    "cfg5s": dict(desc="500 relations, linear/cos/logistic, dim 256, 2M entities, B=2000, 100 batch + 100 uniform negatives, single-relation batches",
                  entities=2_000_000, edges=4_000_000, dim=256, batch=2000, batch_negs=100, uniform_negs=100,
                  operator="linear", comparator="cos", loss="logistic", relations=500, dynamic=False,
                  init_scale=1e-3, zipf=None, rel_zipf=1.2, two_tables=False),
    "cfg2d": dict(desc="1345 relations (dynamic: one per edge), complex_diagonal/dot/softmax, dim 400, 14951 entities, B=1000, chunk 50 + 1000 uniform negatives",
                  entities=14_951, edges=483_142, dim=400, batch=1000, batch_negs=50, uniform_negs=1000,
                  operator="complex_diagonal", comparator="dot", loss="softmax", relations=1345, dynamic=True,
                  init_scale=1e-3, zipf=1.1, two_tables=False),
    "cfg2cos": dict(desc="the reference's default comparator with a wide negative set: no operator, cos/softmax, dim 400, 14951 entities, B=1000, chunk 50 + 1000 uniform negatives",
                    entities=14_951, edges=483_142, dim=400, batch=1000, batch_negs=50, uniform_negs=1000,
                    operator="none", comparator="cos", loss="softmax", relations=1, dynamic=False,
                    init_scale=1e-3, zipf=1.1, two_tables=False),
    "cfg1cos": dict(desc="cfg1 with the reference's default comparator: single relation, identity/cos/ranking(0.1), dim 100, 100k entities, B=1000, 50 batch + 50 uniform negatives",
                    entities=100_000, edges=1_000_000, dim=100, batch=1000, batch_negs=50, uniform_negs=50,
                    operator="none", comparator="cos", loss="ranking", relations=1, dynamic=False,
                    init_scale=1e-3, zipf=None, two_tables=False),
    "livejournal": dict(desc="the reference's LiveJournal example as configured (examples/configs/livejournal_config.py): single relation, identity/cos/ranking(0.1), dim 1024, 4.85M entities, B=1000, 50 batch + 50 uniform negatives",
                        entities=4_847_571, edges=4_000_000, dim=1024, batch=1000, batch_negs=50, uniform_negs=50,
                        operator="none", comparator="cos", loss="ranking", relations=1, dynamic=False,
                        init_scale=1e-3, zipf=2.0, two_tables=False),
    "d400": dict(desc="cfg2's table and operator with the reference's default negatives: complex_diagonal/dot/softmax, dim 400, 14951 entities, B=1000, 50 batch + 50 uniform negatives, single-relation batches",
                 entities=14_951, edges=483_142, dim=400, batch=1000, batch_negs=50, uniform_negs=50,
                 operator="complex_diagonal", comparator="dot", loss="softmax", relations=1345, dynamic=False,
                 init_scale=1e-3, zipf=1.1, two_tables=False),
    "d256dot": dict(desc="no operator, dot/softmax, dim 256, 14951 entities, B=1000, 50 batch + 50 uniform negatives (taken by both the sliced chunk kernel and the streaming route)",
                    entities=14_951, edges=483_142, dim=256, batch=1000, batch_negs=50, uniform_negs=50,
                    operator="none", comparator="dot", loss="softmax", relations=1, dynamic=False,
                    init_scale=1e-3, zipf=1.1, two_tables=False),
    "d400cos": dict(desc="the reference's defaults at dim 400: no operator, cos/ranking(0.1), 100k entities, B=1000, 50 batch + 50 uniform negatives",
                    entities=100_000, edges=1_000_000, dim=400, batch=1000, batch_negs=50, uniform_negs=50,
                    operator="none", comparator="cos", loss="ranking", relations=1, dynamic=False,
                    init_scale=1e-3, zipf=None, two_tables=False),
    "d200transe": dict(desc="TransE at dim 200: translation/l2/ranking(0.1), 100k entities, B=1000, 50 batch + 50 uniform negatives",
                       entities=100_000, edges=1_000_000, dim=200, batch=1000, batch_negs=50, uniform_negs=50,
                       operator="translation", comparator="l2", loss="ranking", relations=1, dynamic=False,
                       init_scale=1e-3, zipf=None, two_tables=False),
    "d200": dict(desc="as d400 at dim 200",
                 entities=14_951, edges=483_142, dim=200, batch=1000, batch_negs=50, uniform_negs=50,
                 operator="complex_diagonal", comparator="dot", loss="softmax", relations=1345, dynamic=False,
                 init_scale=1e-3, zipf=1.1, two_tables=False),
    "fb15k": dict(desc="the reference's FB15k example as configured (examples/configs/fb15k_config_cpu.py): 1345 relations (dynamic), complex_diagonal/dot/softmax, dim 400, 14951 entities, B=1000, chunk 50 + 1000 uniform negatives, N3 regularizer 1e-3",
                  entities=14_951, edges=483_142, dim=400, batch=1000, batch_negs=50, uniform_negs=1000,
                  operator="complex_diagonal", comparator="dot", loss="softmax", relations=1345, dynamic=True,
                  init_scale=1e-3, zipf=1.1, two_tables=False, regularization_coef=1e-3),
}

# batches timed per workload when --steps is not given (a call is `workers` of them)
DEFAULT_BATCHES = {"cfg1": 64000, "cfg1cos": 64000, "cfg2": 400, "cfg2b": 1600, "cfg2d": 400, "cfg2cos": 400, "fb15k": 400,
                   "d400": 6400, "d200": 6400, "d256dot": 6400, "d400cos": 6400, "d200transe": 6400, "livejournal": 3200,
                   "cfg3": 40, "cfg3-hot": 40, "cfg4": 32000, "cfg5": 400, "cfg5s": 800}
# the configurations reported under "configs" beside the cfg1 line, with (timed calls, warm-up calls, CPU seconds)
EXTRA_CONFIGS = {"cfg2": (10, 2, 4.0), "cfg2d": (10, 2, 4.0), "cfg2b": (10, 2, 4.0), "cfg2cos": (10, 2, 4.0), "cfg3": (3, 1, 5.0),
                 "cfg3-hot": (3, 1, 0.0), "cfg4": (100, 10, 4.0), "cfg5": (10, 2, 4.0)}


def power_law_ids(n, num, s, gen, device):
    """ids in [0, num) with P(rank r) ~ r^-s, ranks mapped through a shuffle."""
    u = torch.rand(n, generator=gen, device=device, dtype=torch.float64)
    if abs(s - 1.0) < 1e-9:
        r = torch.exp(u * math.log(num))
    else:
        a = 1.0 - s
        r = ((num ** a - 1.0) * u + 1.0) ** (1.0 / a)
    ranks = (r.floor().long() - 1).clamp_(0, num - 1)
    shuffle = torch.randperm(num, generator=gen, device=device)
    return shuffle[ranks]


def capped_power_law_degrees(num, s, lo, cap, gen, device):
    """`num` i.i.d. integers with P(k) ~ k^-s on lo <= k <= cap (inverse of the exact discrete CDF)."""
    k = torch.arange(lo, cap + 1, dtype=torch.float64, device=device)
    cdf = torch.cumsum(k ** -s, 0)
    cdf = cdf / cdf[-1].clone()
    u = torch.rand(num, generator=gen, device=device, dtype=torch.float64)
    return torch.searchsorted(cdf, u).clamp_(max=cap - lo) + lo


def preferential_attachment_targets(n, num, gen, device):
    """Targets of n edges by preferential attachment on the total degree (the Barabasi-Albert rule), returned in
    shuffled order.  The entities arrive at a constant rate over the edge sequence (n_t = ceil((t + 1) * num / n)
    of them are there for edge t), each with its mean out-degree m = n / num already counted, and edge t names
    v < n_t with probability ~ in-degree(v) so far + m: with probability t / (t + m * n_t) it copies the target of
    a uniformly chosen earlier edge (which names v with probability in-degree(v) / t), otherwise it names a
    uniformly chosen arrived entity.  An entity that arrives at edge t_v ends with about m * sqrt(n / t_v)
    in-edges: the model's power law of exponent 3, the largest in-degree about m * sqrt(num).  The copies form a
    forest over the edges, resolved by pointer jumping."""
    t = torch.arange(n, device=device, dtype=torch.float64)
    arrived = torch.ceil((t + 1.0) * (num / n)).clamp_(1, num)
    copies = torch.rand(n, generator=gen, device=device, dtype=torch.float64) * (t + (n / num) * arrived) < t
    earlier = (torch.rand(n, generator=gen, device=device, dtype=torch.float64) * t).long()
    own = torch.arange(n, device=device)
    parent = torch.where(copies, torch.minimum(earlier, (own - 1).clamp_(min=0)), own)
    fresh = (torch.rand(n, generator=gen, device=device, dtype=torch.float64) * arrived).long().clamp_(max=num - 1)
    del t, copies, earlier, arrived
    while True:
        nxt = parent[parent]
        if torch.equal(nxt, parent):
            break
        parent = nxt
    # entity numbers say nothing about arrival order afterwards, and neither does the position in the list
    relabel = torch.randperm(num, generator=gen, device=device)
    return relabel[fresh[parent]][torch.randperm(n, generator=gen, device=device)]


def livejournal_like_edges(entities, edges, s, cap, gen, device):
    """cfg3's graph as BASELINE.json states it: every entity draws an out-degree from P(k) ~ k^-s on
    2 <= k <= cap (the support starts at 2 because that is what makes 4.85M sources carry 69M edges:
    mean 14.7 against the 14.2 asked for), a uniformly chosen subset of exactly `edges` of those edge
    slots is kept in shuffled order (the trainer shuffles a bucket's edges anyway), and the targets come
    from preferential attachment on the total degree (in-degree power law of exponent 3)."""
    deg = capped_power_law_degrees(entities, s, 2, cap, gen, device)
    src = torch.repeat_interleave(torch.arange(entities, device=device), deg)
    total = src.shape[0]
    if total >= edges:
        pick = torch.randperm(total, generator=gen, device=device)[:edges]
    else:  # only for small samples of the generator
        pick = torch.randint(0, total, (edges,), generator=gen, device=device)
    lhs = src[pick]
    del src, pick
    rhs = preferential_attachment_targets(edges, entities, gen, device)
    return lhs, rhs


def make_workload(w, device, seed=0):
    gen = torch.Generator(device=device).manual_seed(seed)
    e, d = w["entities"], w["dim"]
    tables = [torch.randn(e, d, generator=gen, device=device) * w["init_scale"]]
    if w["two_tables"]:
        tables.append(torch.randn(e, d, generator=gen, device=device) * w["init_scale"])
    n = w["edges"]
    if w.get("graph") == "livejournal":
        lhs, rhs = livejournal_like_edges(e, n, w["zipf"], w["degree_cap"], gen, device)
    elif w["zipf"]:
        lhs = power_law_ids(n, e, w["zipf"], gen, device)
        rhs = power_law_ids(n, e, w["zipf"], gen, device)
    else:
        lhs = torch.randint(0, e, (n,), generator=gen, device=device)
        rhs = torch.randint(0, e, (n,), generator=gen, device=device)
    return tables, lhs, rhs


def host_cores():
    host = os.cpu_count() or 1
    return host, min(host, int(os.environ.get("OMP_NUM_THREADS", host)), 16)  # a GPU box grants 16 host cores per GPU


def cpu_baseline(w, seconds):
    """PBG's train_cpu HOGWILD loop (oracle.hogwild) on this box's host cores,
    on a bounded sample of the same synthetic workload."""
    from oracle import hogwild, step as ostep

    host, cores = host_cores()
    b, d = w["batch"], w["dim"]
    sample = dict(w)
    sample["entities"] = min(w["entities"], 2_000_000, int(2e9) // (4 * d))  # bounded host copy of the table (2 GB)
    sample["edges"] = min(w["edges"], max(cores * 8 * b, 200_000))
    tables, lhs, rhs = make_workload(sample, torch.device("cpu"))
    gen = torch.Generator().manual_seed(1)
    n = lhs.shape[0]
    if w["relations"] > 1:
        s = w.get("rel_zipf") or w["zipf"]
        pool = power_law_ids(4096, w["relations"], s, gen, "cpu") if s else torch.randint(0, w["relations"], (4096,), generator=gen)
    else:
        pool = torch.zeros(4096, dtype=torch.int64)
    rel = pool[torch.arange(n) // b % 4096]
    if w["dynamic"]:
        s_rel = w.get("rel_zipf") or w["zipf"]
        rel = power_law_ids(n, w["relations"], s_rel, gen, "cpu") if s_rel else torch.randint(0, w["relations"], (n,), generator=gen)
    cfg = ostep.StepConfig(dim=d, operator=w["operator"], comparator=w["comparator"], loss=w["loss"], margin=0.1,
                           num_batch_negs=w["batch_negs"], num_uniform_negs=w["uniform_negs"], dynamic=w["dynamic"],
                           num_relations=w["relations"], lr=0.1, relation_weights=[1.0] * w["relations"],
                           regularization_coef=w.get("regularization_coef", 0.0))
    eps, edges, wall = hogwild.run(cfg, tables[0], lhs, rhs, rel, b, cores, seconds,
                                   w_rhs=tables[1] if len(tables) > 1 else None)
    note = "" if sample["entities"] == w["entities"] else f", the generator run for {sample['entities']} entities and {sample['edges']} edges"
    return {"value": eps, "unit": "edges/s", "cores": cores, "host_cpu_count": host, "kind": "port",
            "sample": f"{edges} edges in {wall:.1f} s, {cores} HOGWILD processes over shared-memory tables (oracle.hogwild){note}"}


def algorithmic(w, spec):
    """Per-batch algorithmic bytes and flops of each stage."""
    b, d = w["batch"], w["dim"]
    p, c, u = spec.chunk_size, spec.num_chunks, w["uniform_negs"]
    n = (p if w["batch_negs"] > 0 else 0) + u
    rows = 2 * b + 2 * c * u
    gemm = 2.0 * 2 * c * p * n * d  # both sides, multiply-add
    out = {
        "prep": ("hbm", rows * (2 * 4 * d + 8)),          # gather: read row, write row, read index
        "scores": ("mfma", gemm),
        "loss": ("hbm", 2 * 2 * c * p * n * 4),           # read S, write dS, both sides
        "backward_dn": ("mfma", gemm),
        "backward_da": ("mfma", gemm),
        "rowback": ("hbm", rows * (3 * 4 * d)),           # read prepared grad + prepared row, write raw grad
        "sort": ("hbm", rows * 12 * 2),
        "update": ("hbm", rows * (3 * 4 * d + 8) + rows * 8),  # grad read + W read/write + G r/w + key (duplicates not credited)
    }
    if w["operator"] == "linear":
        op_rows = 2 * b if w["dynamic"] else b + c * u
        out["operator"] = ("mfma", 2.0 * op_rows * d * d)
        out["params"] = ("mfma", 2.0 * 2 * op_rows * d * d)
    # The LDS-resident chunk kernel does gather, operator, scores, loss, backward
    # and the chain rule in one launch: forward + 2 x backward multiply-adds of the
    # positive pairs and of both score matrices.  Its arithmetic intensity
    # (flops / (rows read once + gradient rows written once)) is above the
    # machine balance of 157.3 TFLOP/s : 8 TB/s = 20 flop/byte, so the matrix
    # cores are the roofline that bounds it.
    out["fused_chunk"] = ("mfma", 3 * 2.0 * (b * d + 2 * c * p * n * d))
    out["fused_chunk_bytes"] = rows * (2 * 4 * d + 8) + 3 * b * 8
    # The streaming chunk kernel (positives in LDS, negatives streamed past them twice): the three products of
    # both sides, every score matrix with the chunk's P own rows as its first columns (their diagonal carries
    # the positive pair).  Its HBM side: every negative's raw row read in both sweeps (from the table, by id),
    # its gradient row written once, the positives' operand rows read and their gradients written.
    ns = p + u
    out["stream_chunk"] = ("mfma", 3 * 2.0 * 2 * c * p * ns * d)
    out["stream_chunk_bytes"] = 2 * c * ns * (3 * 4 * d + 4) + 2 * b * (3 * 4 * d)
    return out


def event_timer(reps):
    """median seconds of `reps` calls of fn, each bracketed by events on torch's current stream
    (the stand-alone entry points enqueue on the stream they are handed, which is that one)"""
    def timed(fn, n=reps):
        # warm-up: at least one call, and the device kept busy for 0.1 s (a handful of millisecond launches
        # are over before the clocks have settled)
        t0 = time.perf_counter()
        while True:
            fn()
            torch.cuda.synchronize()
            if time.perf_counter() - t0 > 0.1:
                break
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
        ev[0].record()
        for i in range(n):
            fn()
            ev[i + 1].record()
        torch.cuda.synchronize()
        ts = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(n))
        return ts[len(ts) // 2] * 1e-3
    return timed


def standalone_kernels(pkg):
    """Achieved HBM bandwidth of the stand-alone gather (pbg_gather_rows) and sparse
    RowAdagrad step (pbg_row_adagrad_sparse) on tables far larger than the 256 MB
    Infinity Cache, random indices.  Algorithmic bytes: gather n * (2 * 4D + 8);
    update unique * (2 * 4D + 8) + n * (4D + 8) (table rows read and written, sums,
    every gradient row and index read once).  At D = 100 a 400-byte row straddles
    four 128-byte lines whatever its offset, so `line_granular_ceiling_frac` gives
    what a kernel moving whole lines at the device copy's rate would reach."""
    lib = pkg._lib.lib()
    dev = torch.device("cuda:0")
    stream = lambda: torch.cuda.current_stream().cuda_stream
    timed = event_timer(20)

    out = []
    for rows, n, d in ((8_000_000, 4_000_000, 100), (8_000_000, 4_000_000, 128), (1_000_000, 1_000_000, 1024)):
        table = torch.randn(rows, d, device=dev)
        idx = torch.randint(0, rows, (n,), device=dev)
        dst = torch.empty(n, d, device=dev)
        flag = torch.zeros(1, dtype=torch.int32, device=dev)
        t = timed(lambda: lib.pbg_gather_rows(table.data_ptr(), rows, d, idx.data_ptr(), n, dst.data_ptr(),
                                              flag.data_ptr(), stream()))
        m = min(n, rows)
        t_copy = timed(lambda: dst[:m].copy_(table[:m]))
        gsum = torch.zeros(rows, device=dev)
        grad = torch.randn(n, d, device=dev)
        nbytes = lib.pbg_row_adagrad_sparse_workspace_bytes(n)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        t_upd = timed(lambda: lib.pbg_row_adagrad_sparse(table.data_ptr(), gsum.data_ptr(), rows, d, idx.data_ptr(),
                                                         grad.data_ptr(), n, 0.1, ws.data_ptr(), nbytes, stream()), 10)
        unique = int(torch.unique(idx).numel())
        gather_bytes = n * (2 * 4 * d + 8)
        update_bytes = unique * (2 * 4 * d + 8) + n * (4 * d + 8)
        copy_gbs = m * d * 8 / t_copy / 1e9
        # lines touched per random row: ceil((offset + 4D) / 128) averaged over the row offsets of a packed table
        row_b = 4 * d
        offs = [(i * row_b) % 128 for i in range(32)]
        lines = sum(-(-(o + row_b) // 128) for o in offs) / len(offs) * 128 / row_b
        gather_amp = (lines + 1.0) / 2.0                              # random row reads, sequential row writes
        upd_rand, upd_seq = unique * 2 * row_b, n * row_b           # table rows read + written at random, gradient rows in order
        update_amp = (upd_rand * lines + upd_seq) / (upd_rand + upd_seq)
        out.append({"table_rows": rows, "indices": n, "unique": unique, "dim": d,
                    "gather_GBs": gather_bytes / t / 1e9, "gather_frac_of_8TBs": gather_bytes / t / 1e9 / HBM_PEAK_GBS,
                    "update_GBs": update_bytes / t_upd / 1e9, "update_frac_of_8TBs": update_bytes / t_upd / 1e9 / HBM_PEAK_GBS,
                    "gather_ms": t * 1e3, "update_ms": t_upd * 1e3,
                    "device_copy_GBs": copy_gbs,
                    "line_granular_ceiling_frac": {"gather": copy_gbs / gather_amp / HBM_PEAK_GBS,
                                                   "update": copy_gbs / update_amp / HBM_PEAK_GBS}})
        del table, dst, grad, gsum, ws
    return {"metric": "stand-alone gather / RowAdagrad update, achieved HBM GB/s", "peak_GBs": HBM_PEAK_GBS,
            "update_includes": "key generation, radix sort, duplicate summation, row update", "cases": out}


def perm_kernels(pkg, small=False):
    """Achieved HBM bandwidth of the permutation helpers on cfg4's sizes (41.65M entities in 4 partitions of
    10.4M rows, one bucket of 91.8M edges split 8 x 8).  Algorithmic bytes: reverse_permutation 16 per entry
    (id read, position written); shuffle_rows (in place: scatter into the scratch and copy back) and shuffle_rows_out
    (into a second buffer) 2 * row + 8 per row; randperm 8 per entry (the output alone);
    sub_bucket 64 per edge (three ids read, two permutation entries looked up, three ids written)."""
    nat = pkg.native
    lib = pkg._lib.lib()
    dev = torch.device("cuda:0")
    timed = event_timer(10)
    scale = 16 if small else 1
    n_ent, n_part, n_edges = 41_652_230 // scale, 10_413_058 // scale, 91_772_824 // scale
    out = {}
    perm = nat.randperm(n_ent, 1, dev)
    t = timed(lambda: nat.reverse_permutation(perm))
    out["reverse_permutation"] = {"n": n_ent, "ms": t * 1e3, "GBs": n_ent * 16 / t / 1e9}
    ws = torch.empty(lib.pbg_randperm_workspace_bytes(n_ent), dtype=torch.uint8, device=dev)
    res = torch.empty(n_ent, dtype=torch.int64, device=dev)
    t = timed(lambda: lib.pbg_randperm(n_ent, 7, res.data_ptr(), ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream))
    out["randperm"] = {"n": n_ent, "ms": t * 1e3, "GBs": n_ent * 8 / t / 1e9}
    del perm, ws, res
    for rows, d in ((n_part, 100), (2_000_000 // scale, 1024), (n_part, 1)):
        tab = torch.randn(rows, d, device=dev) if d > 1 else torch.randn(rows, device=dev)
        p = nat.randperm(rows, 3, dev)
        scratch = torch.empty(rows * d * 4, dtype=torch.uint8, device=dev)
        t = timed(lambda: nat.shuffle_rows(tab, p, scratch))
        out[f"shuffle_rows_{rows}x{d}"] = {"rows": rows, "row_bytes": 4 * d, "ms": t * 1e3,
                                           "GBs": rows * (8 * d + 8) / t / 1e9}
        dst = scratch.view(torch.float32).view(tab.shape)
        t = timed(lambda: nat.shuffle_rows_out(tab, p, dst))
        out[f"shuffle_rows_out_{rows}x{d}"] = {"rows": rows, "row_bytes": 4 * d, "ms": t * 1e3,
                                               "GBs": rows * (8 * d + 8) / t / 1e9}
        del tab, p, scratch, dst
    parts = 8
    lhs = torch.randint(0, n_part, (n_edges,), device=dev)
    rhs = torch.randint(0, n_part, (n_edges,), device=dev)
    rel = torch.zeros(n_edges, dtype=torch.int64, device=dev)
    lp, rp = nat.randperm(n_part, 11, dev), nat.randperm(n_part, 12, dev)
    size = -(-n_part // parts)
    outs = [torch.empty_like(lhs) for _ in range(3)]
    t = timed(lambda: nat.sub_bucket(lhs, rhs, rel, [lp], [rp], [size], [size], parts, parts, False, *outs))
    out["sub_bucket"] = {"edges": n_edges, "parts": f"{parts}x{parts}", "ms": t * 1e3, "GBs": n_edges * 64 / t / 1e9}
    for v in out.values():
        v["frac_of_8TBs"] = v["GBs"] / HBM_PEAK_GBS
    # The same launches priced in the 128-byte lines they move: an 8-byte access at a random place is a whole line.
    # reverse_permutation: the id read in order + one line per position written; sub_bucket: 48 bytes per edge in
    # order + two permutation look-ups of one line each.
    for name, per_item, count in (("reverse_permutation", 8 + 128, n_ent), ("sub_bucket", 48 + 2 * 128, n_edges)):
        v = out[name]
        v["line_granular_GBs"] = count * per_item / (v["ms"] * 1e-3) / 1e9
        v["line_granular_frac_of_8TBs"] = v["line_granular_GBs"] / HBM_PEAK_GBS
    return {"metric": "permutation helpers, achieved HBM GB/s on algorithmic bytes", "peak_GBs": HBM_PEAK_GBS,
            "note": "shuffle_rows and sub_bucket include the host read of their error flag (one synchronisation per call); "
                    "randperm is arithmetic (a keyed bijection per entry), priced here on the 8 bytes it writes",
            "cases": out}


def perm_kernels_cpu(threads):
    """The reference's own util.cpp (compiled into oracle/_ref by oracle/Makefile, present in the build
    container only) on the same sizes, `threads` threads: the CPU baseline of the permutation helpers."""
    import glob
    import importlib.util
    hits = sorted(glob.glob(os.path.join(ROOT, "oracle", "_ref", "_C*.so")))
    if not hits:
        return None
    spec = importlib.util.spec_from_file_location("_C", hits[0])
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)

    def timed(fn, reps=3):
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2]

    n_ent, n_part, n_edges = 41_652_230, 10_413_058, 91_772_824
    out = {}
    t = timed(lambda: ref.randperm(n_ent, threads, 7))
    out["randperm"] = {"n": n_ent, "ms": t * 1e3, "GBs": n_ent * 8 / t / 1e9}
    perm = ref.randperm(n_ent, threads, 7)
    t = timed(lambda: ref.reverse_permutation(perm, threads))
    out["reverse_permutation"] = {"n": n_ent, "ms": t * 1e3, "GBs": n_ent * 16 / t / 1e9}
    del perm
    for rows, d in ((n_part, 100), (2_000_000, 1024), (n_part, 1)):
        tab = torch.randn(rows, d) if d > 1 else torch.randn(rows)
        p = ref.randperm(rows, threads, 3)
        t = timed(lambda: ref.shuffle(tab, p, threads))
        out[f"shuffle_rows_{rows}x{d}"] = {"rows": rows, "row_bytes": 4 * d, "ms": t * 1e3, "GBs": rows * (8 * d + 8) / t / 1e9}
        del tab, p
    parts = 8
    lhs = torch.randint(0, n_part, (n_edges,))
    rhs = torch.randint(0, n_part, (n_edges,))
    rel = torch.zeros(n_edges, dtype=torch.int64)
    lp, rp = ref.randperm(n_part, threads, 11), ref.randperm(n_part, threads, 12)
    outs = [torch.empty_like(lhs) for _ in range(3)]
    t = timed(lambda: ref.sub_bucket(lhs, rhs, rel, [n_part], [lp], [n_part], [rp], *outs, parts, parts, threads, False))
    out["sub_bucket"] = {"edges": n_edges, "parts": f"{parts}x{parts}", "ms": t * 1e3, "GBs": n_edges * 64 / t / 1e9}
    return {"kind": "reference", "threads": threads, "cases": out}


def bucket_epoch(pkg, workers, calls_per_bucket, residents=(2, 3, 4)):
    """cfg4 end to end: 4 entity partitions of 10.4M rows in pinned host memory, 16
    buckets in the reference's inside-out order, partitions swapped between
    buckets by pytorch_biggraph_amd.bucket_loop; a bounded number of edges per
    bucket (the real buckets hold about 91.8M each)."""
    bl = pkg.bucket_loop
    w = WORKLOADS["cfg4"]
    nparts, rows, d, b = 4, w["entities"], w["dim"], w["batch"]
    per_bucket = calls_per_bucket * workers * b
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(0)
    t0 = time.perf_counter()
    store = bl.PartitionStore()
    for p in range(nparts):
        store.add(("entity", p), (torch.randn(rows, d, generator=gen, device=dev) * w["init_scale"]).cpu())
    edges = {}
    for lhs in range(nparts):
        for rhs in range(nparts):
            edges[bl.Bucket(lhs, rhs)] = (power_law_ids(per_bucket, rows, w["zipf"], gen, dev),
                                          power_law_ids(per_bucket, rows, w["zipf"], gen, dev),
                                          torch.zeros(per_bucket, dtype=torch.int64, device=dev))
    setup_s = time.perf_counter() - t0
    results = {}
    for resident in residents:
        translation = {"translation": torch.zeros(1, d, device=dev)}
        loop = bl.BucketLoop(store, edges, lhs_entity="entity", rhs_entity="entity", nparts_lhs=nparts, nparts_rhs=nparts,
                             dim=d, batch_size=b, num_workers=workers, num_batch_negs=w["batch_negs"],
                             num_uniform_negs=w["uniform_negs"], operator=w["operator"], comparator=w["comparator"],
                             loss=w["loss"], margin=0.1, lr=0.1, rhs_op=translation,
                             rhs_op_sum={"translation": torch.zeros(1, d, device=dev)}, resident_partitions=resident,
                             bucket_order="inside_out", seed=0)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        stats = loop.train_epoch()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        n = sum(s.num_edges for s in stats)
        results[resident] = {"edges_per_s": n / dt, "seconds": dt, "uploaded_GB": loop.cache.bytes_uploaded / 1e9,
                             "written_back_GB": loop.cache.bytes_written_back / 1e9,
                             "mean_loss_per_edge": sum(s.loss for s in stats) / n}
        del loop
    best = results[3] if 3 in results else results[residents[0]]
    calls = 16 * per_bucket // (b * workers)
    return {"value": best["edges_per_s"], "unit": "edges/s", "steps": calls, "ms_per_step": best["seconds"] / max(1, calls) * 1e3,
            "workload": "cfg4-epoch: one pass over 16 buckets of 4 x 4 partitions (10.4M rows x dim 100 each, pinned host "
                        f"memory), {per_bucket} edges per bucket, translation/l2/ranking, partitions swapped between buckets",
            "batch_size": b, "hogwild_workers": workers, "resident_partitions": 3 if 3 in results else residents[0],
            "setup_seconds": setup_s, "partition_swap": {str(k): v for k, v in results.items()}}


class Workload:
    """One workload resident in HBM: tables, edge list, relation ids; `run` times calls of pbg_train_step on it."""

    def __init__(self, pkg, name, half_precision=False, preheat_ms=200.0):
        self.pkg, self.name, self.w = pkg, name, WORKLOADS[name]
        self.half = half_precision
        self.preheat_s = preheat_ms / 1e3
        self.dev = dev = torch.device("cuda:0")
        w = self.w
        self.tables, self.lhs_all, self.rhs_all = make_workload(w, dev)
        self.gen = gen = torch.Generator(device=dev).manual_seed(1)
        n_edges, b = self.lhs_all.shape[0], w["batch"]
        if w["relations"] > 1:
            if w.get("rel_zipf"):
                self.rel_pool = power_law_ids(4096, w["relations"], w["rel_zipf"], gen, dev)
            elif w["zipf"]:
                self.rel_pool = power_law_ids(4096, w["relations"], w["zipf"], gen, dev)
            else:
                self.rel_pool = torch.randint(0, w["relations"], (4096,), generator=gen, device=dev)
        else:
            self.rel_pool = torch.zeros(4096, dtype=torch.int64, device=dev)
        self.rel_edges = None
        if w["dynamic"]:
            # one relation per edge, sorted inside every batch-sized slice ("mixed batches sorted by relation")
            s_rel = w.get("rel_zipf") or w["zipf"]
            rel_edges = power_law_ids(n_edges, w["relations"], s_rel, gen, dev) if s_rel else \
                torch.randint(0, w["relations"], (n_edges,), generator=gen, device=dev)
            full = n_edges // b * b
            rel_edges[:full] = rel_edges[:full].view(-1, b).sort(dim=1).values.reshape(-1)
            self.rel_edges = rel_edges
        self.enqueue_s = 0.0  # host time per call of the last run's timed loop (launches only, no wait)
        self.route_of = {}    # workers -> which kernels pbg_train_step ran ("staged", "fused", "stream")

    def make_runner(self, workers):
        w, pkg, dev = self.w, self.pkg, self.dev
        d, b = w["dim"], w["batch"]
        spec = pkg.StepSpec(dim=d, batch_size=b, num_workers=workers, num_batch_negs=w["batch_negs"],
                            num_uniform_negs=w["uniform_negs"], operator=w["operator"], dynamic=w["dynamic"],
                            num_relations=w["relations"], comparator=w["comparator"], loss=w["loss"], margin=0.1,
                            lr=0.1, regularization_coef=w.get("regularization_coef", 0.0),
                            half_precision=self.half)
        ws = [t.clone() for t in self.tables]
        gs = [torch.zeros(t.shape[0], device=dev) for t in self.tables]
        rhs_op = {}
        r = w["relations"]
        if w["operator"] == "complex_diagonal":
            rhs_op = {"real": torch.ones(r, d // 2, device=dev), "imag": torch.zeros(r, d // 2, device=dev)}
        elif w["operator"] == "translation":
            rhs_op = {"translation": torch.zeros(r, d, device=dev)}
        elif w["operator"] == "diagonal":
            rhs_op = {"diagonal": torch.ones(r, d, device=dev)}
        elif w["operator"] == "linear":
            rhs_op = {"linear_transformation": torch.eye(d, device=dev).repeat(r, 1, 1).contiguous()}
        rhs_sum = {k: torch.zeros_like(v) for k, v in rhs_op.items()}
        lhs_op = {k: v.clone() for k, v in rhs_op.items()} if w["dynamic"] else {}
        lhs_sum = {k: torch.zeros_like(v) for k, v in lhs_op.items()}
        runner = pkg.StepRunner(spec, ws[0], gs[0], ws[1] if len(ws) > 1 else None, gs[1] if len(gs) > 1 else None,
                                rhs_op, rhs_sum, lhs_op, lhs_sum)
        return spec, runner

    def run(self, workers, calls, warm_calls, profile_calls=0, hip_graph=False):
        w, dev, gen = self.w, self.dev, self.gen
        lhs_all, rhs_all, rel_edges, rel_pool = self.lhs_all, self.rhs_all, self.rel_edges, self.rel_pool
        e, b = w["entities"], w["batch"]
        n_edges = lhs_all.shape[0]
        spec, runner = self.make_runner(workers)
        c, u = spec.num_chunks, w["uniform_negs"]
        per_call = workers * b
        n_r = self.tables[-1].shape[0]

        static = None  # inputs of the captured step (hip_graph): the next call's edges and negatives are written into them

        def one_call(i, profiled=False):
            off = (i * per_call) % (n_edges - per_call + 1) // b * b
            if static is not None:
                s_lhs, s_rhs, s_rel, s_ul, s_ur, graph = static
                s_lhs.copy_(lhs_all[off:off + per_call])
                s_rhs.copy_(rhs_all[off:off + per_call])
                if rel_edges is not None:
                    s_rel.copy_(rel_edges[off:off + per_call])
                else:
                    s_rel.copy_(rel_pool[(i * workers) % (4096 - workers + 1):][:workers])
                torch.randint(0, e, (workers, c, u), generator=gen, device=dev, out=s_ul)
                torch.randint(0, n_r, (workers, c, u), generator=gen, device=dev, out=s_ur)
                graph.replay()
                return None
            lhs = lhs_all[off:off + per_call]
            rhs = rhs_all[off:off + per_call]
            if rel_edges is not None:
                rel = rel_edges[off:off + per_call]
            else:
                rel = rel_pool[(i * workers) % (4096 - workers + 1):][:workers]
            # the uniform negatives of model.py:70-75 are drawn inside the step, a fresh seed per call
            if profiled:
                return runner.train_profiled(lhs, rhs, rel, uniform_seed=0x5EED0000 + i)
            runner.train(lhs, rhs, rel, uniform_seed=0x5EED0000 + i)
            return None

        if hip_graph:
            s_in = [torch.zeros(per_call, dtype=torch.int64, device=dev), torch.zeros(per_call, dtype=torch.int64, device=dev),
                    torch.zeros(per_call if rel_edges is not None else workers, dtype=torch.int64, device=dev),
                    torch.zeros((workers, c, u), dtype=torch.int64, device=dev),
                    torch.zeros((workers, c, u), dtype=torch.int64, device=dev)]
            static = (*s_in, runner.capture_train(*s_in))
        if self.preheat_s > 0 and not hip_graph:
            # The device's clocks take some milliseconds of load to settle, and `--steps 20 --warmup 5` would be
            # over before they have: untimed calls on a scratch copy of the state until preheat_s has passed.
            # They do not touch the state that the warm-up and timed calls train.
            _, scratch = self.make_runner(workers)
            t_end = time.perf_counter() + self.preheat_s
            j = 0
            while time.perf_counter() < t_end:
                for _ in range(4):
                    off = (j * per_call) % (n_edges - per_call + 1) // b * b
                    rel = rel_edges[off:off + per_call] if rel_edges is not None else rel_pool[(j * workers) % (4096 - workers + 1):][:workers]
                    scratch.train(lhs_all[off:off + per_call], rhs_all[off:off + per_call], rel, uniform_seed=0x0BAD0000 + j)
                    j += 1
                torch.cuda.synchronize()
            del scratch
            self.preheat_s = 0.0  # once per workload
        for i in range(warm_calls):
            one_call(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(calls):
            one_call(warm_calls + i)
        self.enqueue_s = (time.perf_counter() - t0) / calls
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        stages = None
        if profile_calls:
            acc = None
            for i in range(profile_calls):
                ms = one_call(warm_calls + calls + i, profiled=True)
                acc = ms if acc is None else [a + m for a, m in zip(acc, ms)]
            stages = dict(zip(runner.STAGES, [a / profile_calls for a in acc]))
            if runner.route == "fused":
                # one kernel covers stages "prep" .. "rowback" (the batches' sums of the statistics ride with the update)
                stages = {"fused_chunk": stages["prep"], "params": stages["params"],
                          "sort": stages["sort"], "update": stages["update"]}
            elif runner.route == "stream":
                # per-edge preparation + column ids | the chunk kernel | per-edge finish
                stages = {"stream_prep": stages["prep"], "stream_chunk": stages["scores"], "stream_finish": stages["rowback"],
                          "params": stages["params"], "sort": stages["sort"], "update": stages["update"]}
        loss = float(runner.loss_out.mean().item()) / b
        self.route_of[workers] = runner.route
        return spec, calls * per_call / dt, dt / calls * 1e3, dt, stages, loss

    def roofline(self, spec, stages, workers):
        """The slowest stage's algorithmic units / its HIP-event time (events on the step's own stream)."""
        alg = algorithmic(self.w, spec)
        dominant = max((k for k in stages if k in alg), key=lambda k: stages[k])
        bound, units_per_batch = alg[dominant]
        launches = {"scores": 2, "backward_dn": 2, "backward_da": 2}.get(dominant, 1)
        seconds = stages[dominant] * 1e-3
        units = units_per_batch * workers
        if bound == "hbm":
            achieved, peak, unit = units / seconds / 1e9, HBM_PEAK_GBS, "GB/s"
        else:
            achieved, peak, unit = units / seconds / 1e12, (FP16_MFMA_PEAK_TFLOPS if self.half else FP32_MFMA_PEAK_TFLOPS), "TFLOP/s"
        roofline = {
            "kernel": dominant, "bound": bound, "achieved": achieved, "peak": peak, "unit": unit,
            "frac": achieved / peak, "traffic": TRAFFIC.get((self.name, dominant, workers)), "launches_in_stage": launches,
            "avg_launch_ms": stages[dominant] / launches,
            "stages_ms": stages,
            "all": {k: {"bound": alg[k][0],
                        "achieved": (alg[k][1] * workers / (stages[k] * 1e-3) / (1e9 if alg[k][0] == "hbm" else 1e12)) if stages[k] > 0 else None}
                    for k in stages if k in alg},
        }
        if dominant in ("fused_chunk", "stream_chunk"):
            # the same launch against the other roofline: rows read once + gradient rows written once
            roofline["algorithmic_hbm_gbs"] = alg[dominant + "_bytes"] * workers / seconds / 1e9
        return roofline

    def release(self):
        self.tables = self.lhs_all = self.rhs_all = self.rel_edges = self.rel_pool = None
        torch.cuda.empty_cache()


def measure_extra(pkg, name, workers, calls, warm, cpu):
    """One entry of "configs": the workload at `workers` batches per call, its slowest stage against its
    roofline, and the strictly sequential order (one batch per call)."""
    t0 = time.perf_counter()
    wl = Workload(pkg, name, preheat_ms=100.0)
    spec, eps, ms, wall, stages, loss = wl.run(workers, calls, warm, profile_calls=3)
    roof = wl.roofline(spec, stages, workers)
    seq_calls = 20 if wl.w["batch"] >= 10_000 else 100
    _, seq_eps, seq_ms, _, _, _ = wl.run(1, seq_calls, 5)
    out = {"workload": f"{name}: {wl.w['desc']}", "value": eps, "unit": "edges/s", "ms_per_step": ms, "steps": calls, "warmup": warm,
           "route": wl.route_of[workers], "hogwild_workers": workers, "batch_size": wl.w["batch"],
           "negatives_per_edge_per_side": spec.chunk_size * (wl.w["batch_negs"] > 0) + wl.w["uniform_negs"],
           "mean_loss_per_edge_last_call": loss,
           "roofline": {k: roof[k] for k in ("kernel", "bound", "achieved", "peak", "unit", "frac", "launches_in_stage", "avg_launch_ms", "stages_ms")},
           "sequential_value": seq_eps, "sequential_ms_per_step": seq_ms, "cpu_baseline": cpu,
           "bench_seconds": None}
    wl.release()
    out["bench_seconds"] = time.perf_counter() - t0
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed calls of pbg_train_step (each of --workers batches)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed calls")
    ap.add_argument("--preheat-ms", type=float, default=200.0,
                    help="untimed calls on a scratch copy of the state before the warm-up calls, until this much time has passed")
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS) + ["cfg4-epoch"],
                    help="measure this workload only (default: cfg1 as the line, every other BASELINE configuration under \"configs\")")
    ap.add_argument("--extras", action="store_true", help="with --workload: also run the other configurations and tables")
    ap.add_argument("--no-extras", action="store_true", help="without --workload: cfg1 only")
    ap.add_argument("--configs", default=None, help="comma-separated subset of " + ",".join(EXTRA_CONFIGS) + ",k_sweep,standalone,perm,cfg4-epoch")
    ap.add_argument("--workers", type=int, default=64,
                    help="batches in flight per call (HOGWILD workers); 64 batches of cfg1 are 1280 chunks = 5 per compute unit")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="length of the CPU baseline sample (0 = skip every CPU leg)")
    ap.add_argument("--no-sequential", action="store_true", help="skip the workers=1 measurement")
    ap.add_argument("--half-precision", action="store_true",
                    help="the reference's config.half_precision (dot / cos workloads): float16 embeddings from "
                         "comparator.prepare on, products on the fp16 matrix instructions; never the default line")
    ap.add_argument("--standalone-kernels", action="store_true",
                    help="only measure the stand-alone gather and sparse RowAdagrad kernels on large tables")
    ap.add_argument("--perm-kernels", action="store_true", help="only measure the permutation helpers on cfg4's sizes")
    ap.add_argument("--perm-kernels-cpu", type=int, default=0, metavar="THREADS",
                    help="only time the reference's compiled util.cpp (oracle/_ref, build container only) on the same sizes")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain 1 GiB device copy 5 times (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU (one process, no collectives); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.perm_kernels_cpu:
        print(json.dumps(perm_kernels_cpu(args.perm_kernels_cpu)))
        return
    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "5 device copies", "bytes_read_each": src.numel() * 4, "bytes_written_each": src.numel() * 4}))
        return

    import __graft_entry__

    if args.standalone_kernels:
        print(json.dumps(standalone_kernels(__graft_entry__.load_package())))
        return
    if args.perm_kernels:
        print(json.dumps(perm_kernels(__graft_entry__.load_package())))
        return
    if args.workload == "cfg4-epoch":
        r = bucket_epoch(__graft_entry__.load_package(), args.workers, args.steps or 31)
        line = {"metric": "train edges/sec (100 negs/edge) on 1 MI355X", "value": r["value"], "unit": "edges/s", "n_gpus": 1,
                "steps": r["steps"], "warmup": 0, "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak",
                "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                "config": {k: r[k] for k in ("workload", "batch_size", "hogwild_workers", "resident_partitions", "setup_seconds")},
                "partition_swap": r["partition_swap"], "roofline": None, "cpu_baseline": None}
        print(json.dumps(line))
        return

    name = args.workload or "cfg1"
    with_extras = (args.workload is None and not args.no_extras) or args.extras
    chosen = None if args.configs is None else set(args.configs.split(","))
    extras = [n for n in EXTRA_CONFIGS if n != name and (chosen is None or n in chosen)] if with_extras else []
    tables_wanted = [t for t in ("k_sweep", "standalone", "perm", "cfg4-epoch") if with_extras and (chosen is None or t in chosen)]
    w = WORKLOADS[name]
    t_start = time.perf_counter()
    # The CPU baselines run first, before this process opens the GPU: their worker
    # processes each touch the HIP runtime once (autograd asks it for a device
    # count), and the box allows 16 processes on the card at a time.
    # (the CPU baseline is the reference's CPU path, which has no half precision: fp32 beside either line)
    cpu = cpu_baseline(w, args.cpu_seconds) if args.cpu_seconds > 0 else None
    cpu_extra = {}
    for n in extras:
        secs = EXTRA_CONFIGS[n][2]
        cpu_extra[n] = cpu_baseline(WORKLOADS[n], secs) if args.cpu_seconds > 0 and secs > 0 else None
    cpu_legs_s = time.perf_counter() - t_start

    pkg = __graft_entry__.load_package()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    wl = Workload(pkg, name, half_precision=args.half_precision, preheat_ms=args.preheat_ms)
    b = w["batch"]
    workers = max(1, args.workers)
    default_batches = DEFAULT_BATCHES[name]
    steps = args.steps if args.steps is not None else max(1, default_batches // workers)
    warmup = args.warmup if args.warmup is not None else max(1, steps // 10)
    spec, eps, ms_per_step, wall_s, stages, loss = wl.run(workers, steps, warmup, profile_calls=10)
    host_enqueue_ms = wl.enqueue_s * 1e3
    route = wl.route_of[workers]

    seq = None
    if not args.no_sequential and workers > 1:
        seq_calls = max(50, min(default_batches // 8, 1000))
        _, seq_eps, seq_ms, _, _, _ = wl.run(1, seq_calls, 20)
        seq = {"value": seq_eps, "ms_per_step": seq_ms, "steps": seq_calls, "workers": 1}
        # the same single-batch sequence with the step captured in a HIP graph (one launch per step
        # instead of about ten) and the inputs written into the graph's static buffers
        _, g_eps, g_ms, _, _, _ = wl.run(1, seq_calls, 20, hip_graph=True)
        seq["hip_graph"] = {"value": g_eps, "ms_per_step": g_ms, "steps": seq_calls}

    roofline = wl.roofline(spec, stages, workers)

    k_sweep = None
    if "k_sweep" in tables_wanted:
        # edges/s against the number of batches per call (= the staleness a batch may see, in batches)
        k_sweep = []
        for k in (1, 2, 4, 8, 16, 40, 64):
            calls = max(50, min(default_batches // k, 1000))
            _, k_eps, k_ms, _, _, _ = wl.run(k, calls, 20)
            k_sweep.append({"workers": k, "value": k_eps, "ms_per_step": k_ms, "steps": calls})
    wl.release()

    configs = {}
    for n in extras:
        calls, warm, _ = EXTRA_CONFIGS[n]
        try:
            configs[n] = measure_extra(pkg, n, workers, calls, warm, cpu_extra.get(n))
        except Exception as exc:  # one configuration failing must not cost the line
            configs[n] = {"error": f"{type(exc).__name__}: {exc}"}
    standalone = perms = epoch = None
    try:
        if "standalone" in tables_wanted:
            standalone = standalone_kernels(pkg)
        if "perm" in tables_wanted:
            perms = perm_kernels(pkg)
        torch.cuda.empty_cache()
        if "cfg4-epoch" in tables_wanted:
            epoch = bucket_epoch(pkg, workers, 312, residents=(3,))
    except Exception as exc:
        configs["tables_error"] = f"{type(exc).__name__}: {exc}"

    config = {"workload": f"{name}: {w['desc']}" + (", half_precision" if args.half_precision else ""), "batch_size": b,
              "negatives_per_edge_per_side": spec.chunk_size * (w['batch_negs'] > 0) + w["uniform_negs"],
              "hogwild_workers": workers, "step": f"one pbg_train_step call of {workers} batches", "route": route,
              "timed_calls": steps, "timed_batches": steps * workers, "timed_edges": steps * workers * b,
              "timed_wall_seconds": wall_s, "preheat_ms_on_scratch_state": args.preheat_ms,
              "uniform_negative_draw": "inside the step (Philox4x32-10, one seed per call)",
              "mean_loss_per_edge_last_call": loss, "host_enqueue_ms_per_call": host_enqueue_ms}
    # the other configurations once more as flat numbers (edges/s, fraction of the slowest stage's roofline, CPU edges/s)
    for n, r in configs.items():
        if isinstance(r, dict) and "value" in r:
            config[f"{n}_edges_per_s"] = r["value"]
            config[f"{n}_roofline_frac"] = r["roofline"]["frac"]
            config[f"{n}_roofline_kernel"] = f"{r['roofline']['kernel']} ({r['roofline']['bound']})"
            config[f"{n}_cpu_edges_per_s"] = r["cpu_baseline"]["value"] if r.get("cpu_baseline") else None
    if epoch:
        config["cfg4_epoch_edges_per_s"] = epoch["value"]
        # the epoch's calls are cfg4's calls: its kernels' roofline and the CPU's rate on the same step ride along
        c4 = configs.get("cfg4") or {}
        if "roofline" in c4:
            epoch["roofline_of_the_calls"] = {k: c4["roofline"].get(k) for k in ("kernel", "bound", "achieved", "peak", "unit", "frac")}
            epoch["cpu_baseline_of_the_calls"] = c4.get("cpu_baseline")
            epoch["fraction_of_the_resident_rate"] = epoch["value"] / c4["value"]
    line = {
        "metric": "train edges/sec (100 negs/edge) on 1 MI355X",
        "value": eps, "unit": "edges/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 products, f32 sums (config.half_precision)" if args.half_precision else "f32", "data": "synthetic",
        "config": config,
        "sequential": seq,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    if with_extras:
        line.update({"k_sweep": k_sweep, "configs": configs, "standalone": standalone, "perm_kernels": perms, "cfg4_epoch": epoch,
                     "bench_wall_seconds": {"cpu_legs": cpu_legs_s, "total": time.perf_counter() - t_start}})
    print(json.dumps(line))


if __name__ == "__main__":
    main()

"""Partition swap and the per-bucket training loop on one GPU.

Reference: the bucket loop of ``TrainingCoordinator.train``
(torchbiggraph/train_cpu.py:592-714), ``_swap_partitioned_embeddings``
(:789-847), ``_coordinate_train`` (:849-884) and the bucket orders of
torchbiggraph/bucket_scheduling.py:72-262.

The reference keeps exactly the two partitions of the current bucket in memory
and goes through checkpoint files for the rest.  Here every partition's
embedding table and RowAdagrad sum live in PINNED HOST memory
(`PartitionStore`); `PartitionCache` keeps as many of them resident in HBM as
it is given buffers for, writes a partition back only when its buffer is needed
for another one, and loads the next bucket's partitions on a copy stream while
the current bucket trains.  With 288 GB of HBM a whole graph often stays
resident after the first pass and the swap degenerates to nothing; two buffers
reproduce the reference's behaviour.

Edges of a bucket hold partition-local entity offsets, as the reference's edge
files do.  A bucket is trained by `pbg_train_step` calls of `num_workers`
batches each (native.StepRunner); the tail of a bucket runs as one call of the
remaining full batches and one call of the final partial batch
(batching.py:109-112).  With `eval_fraction` a random sample of each bucket's
edges is held out of training and ranked before and after the bucket is trained
(train_cpu.py:648-693).  Standard (non-dynamic) relations are trained in
single-relation batches, the relation of the next batch drawn in proportion to
the edges each relation has left (batching.py:60-79).
"""
import random
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from . import native
from .eval import ranking_stats_from_ranks
from .losses import LOSS_FUNCTIONS
from .stats import Stats
from .util import round_up_to_nearest_multiple

PartitionKey = Tuple[str, int]  # (entity type, partition)


@dataclass(frozen=True)
class Bucket:
    """types.py: Bucket(lhs, rhs) partition pair."""

    lhs: int
    rhs: int

    def __str__(self) -> str:
        return f"( {self.lhs} , {self.rhs} )"


def create_buckets_ordered_lexicographically(nparts_lhs: int, nparts_rhs: int) -> List[Bucket]:
    """Increasing LHS and, for the same LHS, increasing RHS (bucket_scheduling.py:91-98)."""
    return [Bucket(lhs, rhs) for lhs in range(nparts_lhs) for rhs in range(nparts_rhs)]


def create_buckets_ordered_randomly(nparts_lhs: int, nparts_rhs: int, *, generator: random.Random) -> List[Bucket]:
    """bucket_scheduling.py:101-111."""
    buckets = create_buckets_ordered_lexicographically(nparts_lhs, nparts_rhs)
    generator.shuffle(buckets)
    return buckets


def create_layer_of_buckets(nparts_lhs: int, nparts_rhs: int, layer_idx: int, *, generator: random.Random) -> List[Bucket]:
    """Layer i: the buckets with min(lhs, rhs) == i, shuffled (bucket_scheduling.py:203-219)."""
    layer = [Bucket(layer_idx, layer_idx)]
    layer += [Bucket(lhs, layer_idx) for lhs in range(layer_idx + 1, nparts_lhs)]
    layer += [Bucket(layer_idx, rhs) for rhs in range(layer_idx + 1, nparts_rhs)]
    generator.shuffle(layer)
    return layer


def create_buckets_ordered_by_layer(nparts_lhs: int, nparts_rhs: int, order: str, *,
                                    generator: random.Random) -> List[Bucket]:
    """Concentric L-shaped layers, ``outside_in`` from layer 0 or ``inside_out``
    from the innermost layer (bucket_scheduling.py:222-262)."""
    if order not in ("inside_out", "outside_in"):
        raise ValueError("Unknown order: %s" % order)
    layers = [create_layer_of_buckets(nparts_lhs, nparts_rhs, i, generator=generator)
              for i in range(min(nparts_lhs, nparts_rhs))]
    if order == "inside_out":
        layers.reverse()
    return [b for layer in layers for b in layer]


def create_ordered_buckets(nparts_lhs: int, nparts_rhs: int, order: str, *, generator: random.Random) -> List[Bucket]:
    """bucket_scheduling.py:72-88 (``affinity`` is not provided)."""
    if order == "lexicographic":
        return create_buckets_ordered_lexicographically(nparts_lhs, nparts_rhs)
    if order == "random":
        return create_buckets_ordered_randomly(nparts_lhs, nparts_rhs, generator=generator)
    if order in ("inside_out", "outside_in"):
        return create_buckets_ordered_by_layer(nparts_lhs, nparts_rhs, order, generator=generator)
    raise NotImplementedError("Unknown bucket order: %s" % order)


def holdout_indices(num_edges: int, eval_fraction: float, bucket: Bucket, edge_path_idx: int = 0,
                    edge_chunk_idx: int = 0) -> Optional[torch.Tensor]:
    """The edges of a bucket that are held out for evaluation: int(num_edges *
    eval_fraction) draws WITH replacement from a generator seeded by what
    identifies the edge set, so every epoch holds out the same ones
    (train_cpu.py:648-672).  None when nothing is held out."""
    num_eval = int(num_edges * eval_fraction)
    if num_eval <= 0:
        return None
    g = torch.Generator()
    g.manual_seed(hash((edge_path_idx, edge_chunk_idx, bucket.lhs, bucket.rhs)))
    return torch.randint(num_edges, (num_eval,), dtype=torch.long, generator=g)


def train_edge_indices(num_edges: int, eval_edge_idxs: Optional[torch.Tensor], device=None) -> torch.Tensor:
    """The edges a bucket is trained on, before shuffling (train_cpu.py:852-856):
    position e of [0, num_edges) holds e, except that held-out position
    eval_edge_idxs[j] holds num_train + j; the first num_train positions are kept.
    A held-out edge drawn more than once keeps its LAST j, which is what the
    reference's sequential index assignment leaves (here: a scatter that keeps the
    largest value, so that the result does not depend on the order in which a GPU
    applies the writes).  As in the reference, a held-out edge whose own number is
    num_train + j for a j that was swapped in (e.g. 10 edges, [2, 8] held out: slot
    2 receives 8) is trained on all the same; the statement is kept as it is so
    that the same edges are trained."""
    if eval_edge_idxs is None:
        return torch.arange(num_edges, device=device)
    num_train = num_edges - eval_edge_idxs.shape[0]
    idx = eval_edge_idxs.to(device)
    out = torch.arange(num_edges, device=device)
    out.scatter_reduce_(0, idx, torch.arange(num_train, num_edges, device=device), reduce="amax", include_self=False)
    return out[:num_train]


def plan_relation_batches(group_sizes: Sequence[int], batch_size: int,
                          generator: Optional[torch.Generator] = None) -> List[Tuple[int, int, int]]:
    """The batches batch_edges_group_by_relation_type yields (batching.py:60-79),
    as (group, offset inside the group, length): the group of the next batch is
    drawn with probability proportional to the edges the groups have left, and a
    batch is the group's next batch_size edges (fewer at the group's end)."""
    left = torch.tensor(list(group_sizes), dtype=torch.long)
    plan: List[Tuple[int, int, int]] = []
    while int(left.sum()) > 0:
        idx = int(torch.multinomial(left.float(), 1, generator=generator))
        offset = int(group_sizes[idx]) - int(left[idx])
        length = min(batch_size, int(left[idx]))
        plan.append((idx, offset, length))
        left[idx] -= length
    return plan


class PartitionStore:
    """Every partition's embedding table [rows, dim] and RowAdagrad sum [rows] in
    pinned host memory (the role the checkpoint files play in
    train_cpu.py:813-845)."""

    def __init__(self) -> None:
        self.tables: Dict[PartitionKey, torch.Tensor] = {}
        self.sums: Dict[PartitionKey, torch.Tensor] = {}

    def add(self, key: PartitionKey, table: torch.Tensor, state_sum: Optional[torch.Tensor] = None) -> None:
        if table.dim() != 2 or table.dtype != torch.float32:
            raise TypeError("a partition table must be a 2-dimensional float32 tensor")
        pinned = torch.empty(table.shape, dtype=torch.float32, pin_memory=True)
        pinned.copy_(table)
        sums = torch.zeros(table.shape[0], dtype=torch.float32, pin_memory=True)
        if state_sum is not None:
            sums.copy_(state_sum)
        self.tables[key] = pinned
        self.sums[key] = sums

    def rows(self, key: PartitionKey) -> int:
        return self.tables[key].shape[0]


class _Slot:
    def __init__(self, w: torch.Tensor, g: torch.Tensor) -> None:
        self.w, self.g = w, g
        self.key: Optional[PartitionKey] = None
        self.ready: Optional[torch.cuda.Event] = None     # upload finished (copy stream)
        self.last_use: Optional[torch.cuda.Event] = None  # last training call finished (compute stream)
        self.stamp = 0
        self.dirty = False  # trained on since it was last written back


class PartitionCache:
    """`num_slots` device buffers, each large enough for the largest partition.
    Uploads and write-backs run on their own stream; the training stream waits
    for an upload through an event and the copy stream waits for the last
    training call that touched a buffer before writing it back."""

    def __init__(self, store: PartitionStore, device: torch.device, num_slots: int) -> None:
        if num_slots < 2:
            raise ValueError("at least two partitions must fit (the lhs and rhs partition of a bucket)")
        self.store = store
        self.device = device
        max_rows = max(store.rows(k) for k in store.tables)
        dims = {t.shape[1] for t in store.tables.values()}
        if len(dims) != 1:
            raise ValueError("all partitions must have the same dimension")
        dim = dims.pop()
        self.slots = [_Slot(torch.empty((max_rows, dim), dtype=torch.float32, device=device),
                            torch.empty(max_rows, dtype=torch.float32, device=device)) for _ in range(num_slots)]
        self.by_key: Dict[PartitionKey, _Slot] = {}
        self.copy_stream = torch.cuda.Stream(device=device)  # default priority
        self.clock = 0
        self.bytes_uploaded = 0
        self.bytes_written_back = 0

    def _write_back(self, slot: _Slot) -> None:
        key = slot.key
        n = self.store.rows(key)
        with torch.cuda.stream(self.copy_stream):
            if slot.last_use is not None:
                self.copy_stream.wait_event(slot.last_use)
            self.store.tables[key].copy_(slot.w[:n], non_blocking=True)
            self.store.sums[key].copy_(slot.g[:n], non_blocking=True)
        slot.dirty = False
        self.bytes_written_back += n * (slot.w.shape[1] + 1) * 4

    def _load(self, key: PartitionKey, protected: Sequence[PartitionKey]) -> _Slot:
        free = [s for s in self.slots if s.key is None]
        if free:
            slot = free[0]
        else:
            candidates = [s for s in self.slots if s.key not in protected]
            if not candidates:
                raise RuntimeError("no device buffer left for partition %s" % (key,))
            slot = min(candidates, key=lambda s: s.stamp)  # least recently used
            if slot.dirty:
                self._write_back(slot)
            del self.by_key[slot.key]
        n = self.store.rows(key)
        with torch.cuda.stream(self.copy_stream):
            # a buffer taken over from another partition: its write-back precedes this upload on the same stream
            slot.w[:n].copy_(self.store.tables[key], non_blocking=True)
            slot.g[:n].copy_(self.store.sums[key], non_blocking=True)
            slot.ready = torch.cuda.Event()
            slot.ready.record(self.copy_stream)
        slot.key, slot.last_use, slot.dirty = key, None, False
        self.by_key[key] = slot
        self.bytes_uploaded += n * (slot.w.shape[1] + 1) * 4
        return slot

    def prefetch(self, keys: Sequence[PartitionKey], protected: Sequence[PartitionKey]) -> None:
        """Starts uploading `keys` if buffers can be had without touching `protected`."""
        for key in keys:
            if key in self.by_key:
                continue
            keep = list(protected) + list(keys)
            if all(s.key is not None and s.key in keep for s in self.slots):
                return  # every buffer is spoken for
            self._load(key, keep)

    def acquire(self, keys: Sequence[PartitionKey]) -> List[Tuple[torch.Tensor, torch.Tensor]]:
        """Device views (table, sum) of `keys`, usable on the current stream."""
        out = []
        for key in keys:
            slot = self.by_key.get(key)
            if slot is None:
                slot = self._load(key, keys)
            self.clock += 1
            slot.stamp = self.clock
            torch.cuda.current_stream(self.device).wait_event(slot.ready)
            n = self.store.rows(key)
            out.append((slot.w[:n], slot.g[:n]))
        return out

    def release(self, keys: Sequence[PartitionKey]) -> None:
        """Marks the end of the current stream's work on `keys`."""
        for key in keys:
            slot = self.by_key[key]
            slot.dirty = True
            slot.last_use = torch.cuda.Event()
            slot.last_use.record(torch.cuda.current_stream(self.device))

    def write_back_idle(self, in_use: Sequence[PartitionKey]) -> None:
        """Starts writing back every trained-on partition that the current bucket does not name (the last
        bucket of a pass has no successor to upload for: its idle neighbours go home while it trains)."""
        for slot in self.slots:
            if slot.key is not None and slot.dirty and slot.key not in in_use:
                self._write_back(slot)

    def flush(self) -> None:
        """Writes every resident partition back to the store and waits for it."""
        for slot in self.slots:
            if slot.key is not None and slot.dirty:
                self._write_back(slot)
        self.copy_stream.synchronize()


@dataclass
class BucketStats:
    bucket: Bucket
    num_edges: int
    loss: float
    violators_lhs: int
    violators_rhs: int
    # sums over the held-out edges (divide by .count, or call .average()); None without a hold-out
    eval_before: Optional[Stats] = None
    eval_after: Optional[Stats] = None


class BucketLoop:
    """One pass over all buckets = ``train_epoch()``.

    edges: {Bucket: (lhs, rhs, rel)} int64 tensors of partition-local offsets and
    relation types, on the host (pinned or not) or already on the device.
    """

    def __init__(self, store: PartitionStore, edges: Dict[Bucket, Tuple[torch.Tensor, torch.Tensor, torch.Tensor]],
                 *, lhs_entity: str, rhs_entity: str, nparts_lhs: int, nparts_rhs: int, dim: int, batch_size: int,
                 num_workers: int = 64, num_batch_negs: int = 50, num_uniform_negs: int = 50, operator: str = "none",
                 comparator: str = "dot", loss: str = "ranking", margin: float = 0.1, lr: float = 0.1,
                 relation_lr: Optional[float] = None, dynamic: bool = False, num_relations: int = 1,
                 rhs_op: Optional[Dict[str, torch.Tensor]] = None, rhs_op_sum: Optional[Dict[str, torch.Tensor]] = None,
                 lhs_op: Optional[Dict[str, torch.Tensor]] = None, lhs_op_sum: Optional[Dict[str, torch.Tensor]] = None,
                 resident_partitions: int = 2, bucket_order: str = "inside_out", seed: int = 0,
                 device: str = "cuda:0",
                 regularization_coef: float = 0.0,
                 global_embs: Optional[Dict[str, Tuple[torch.Tensor, torch.Tensor]]] = None,
                 eval_fraction: float = 0.0, eval_num_batch_negs: int = 1000, eval_num_uniform_negs: int = 1000,
                 edge_order: Optional[Callable[[Bucket, int], torch.Tensor]] = None,
                 negatives: Optional[Callable[..., torch.Tensor]] = None,
                 record_calls: bool = False) -> None:
        self.store, self.edges = store, edges
        self.lhs_entity, self.rhs_entity = lhs_entity, rhs_entity
        self.nparts_lhs, self.nparts_rhs = nparts_lhs, nparts_rhs
        self.device = torch.device(device)
        self.batch_size, self.num_workers = batch_size, num_workers
        self.spec_args = dict(dim=dim, num_batch_negs=num_batch_negs, num_uniform_negs=num_uniform_negs,
                              operator=operator, dynamic=dynamic, num_relations=num_relations, comparator=comparator,
                              loss=loss, margin=margin, lr=lr, relation_lr=relation_lr,
                              regularization_coef=regularization_coef)
        # config.global_emb: {entity type: (vector [D], its AsyncAdagrad sum [D])} on the device
        self.global_embs = None
        if global_embs is not None:
            (gl, sl), (gr, sr) = global_embs[lhs_entity], global_embs[rhs_entity]
            self.global_embs = ((gl, gr), (sl, sr))
        self.ops = (rhs_op or {}, rhs_op_sum or {}, lhs_op or {}, lhs_op_sum or {})
        self.cache = PartitionCache(store, self.device, resident_partitions)
        self.bucket_order = bucket_order
        self.rng = random.Random(seed)
        self.generator = torch.Generator(device=self.device).manual_seed(seed)
        self.host_generator = torch.Generator().manual_seed(seed)  # the relation of the next batch
        self.seed = seed
        # edge_order(bucket, n) -> permutation of the bucket's n TRAINING edges, in place
        # of the shuffle of _coordinate_train (train_cpu.py:857-859)
        self.edge_order = edge_order
        # None: the step draws its uniform negatives itself (SimpleEmbedding.sample_entities,
        # model.py:70-75), one seed per call; a callable(workers, chunks, num_uniform, num_rows,
        # generator, device) -> [workers, chunks, num_uniform] supplies them instead
        self.negatives = negatives
        # held-out evaluation (config.py: eval_fraction, eval_num_batch_negs, eval_num_uniform_negs)
        self.eval_fraction = eval_fraction
        self.eval_negs = (eval_num_batch_negs, eval_num_uniform_negs)
        self.loss_fn = LOSS_FUNCTIONS.get_class(loss)(margin=margin)
        # record_calls: keep, on the host, the edges and relation types of every training
        # call (`self.calls_log`), for a caller that wants to replay the epoch elsewhere
        self.calls_log: Optional[List[dict]] = [] if record_calls else None
        self.calls = 0
        self.eval_calls = 0  # seeds of the evaluation's AUC samples
        self.epoch = 0

    def _keys(self, b: Bucket) -> List[PartitionKey]:
        keys = [(self.lhs_entity, b.lhs)]
        if (self.rhs_entity, b.rhs) != keys[0]:
            keys.append((self.rhs_entity, b.rhs))
        return keys

    def _call_plan(self, rel: torch.Tensor, batch_size: int, workers: int, draw: bool):
        """Splits edges (already in training order) into calls of up to `workers`
        equally sized batches.  Returns (order, starts, rels, calls): `order` (or
        None) rearranges the edges so that every batch is a contiguous run,
        batch i covers [starts[i], starts[i] + its length) and has relation
        rels[i] (standard relations only), and calls = [(first batch, number of
        batches, batch length)].

        Dynamic relations, or a single relation type: consecutive batches in the
        given order; the tail runs as one call of the remaining full batches and
        one of the final partial batch.  Standard relations of several types:
        single-relation batches (batching.py:60-79), in drawn order when `draw`,
        else relation by relation."""
        n = rel.shape[0]
        dynamic = self.spec_args["dynamic"]
        if dynamic or self.spec_args["num_relations"] == 1:
            starts = list(range(0, n, batch_size))
            lengths = [min(batch_size, n - s0) for s0 in starts]
            order, rels = None, None
        else:
            sorted_rel, order = torch.sort(rel, stable=True)
            sizes = torch.bincount(rel, minlength=self.spec_args["num_relations"]).tolist()
            present = [r for r, c in enumerate(sizes) if c > 0]
            begin, acc = {}, 0
            for r in present:
                begin[r] = acc
                acc += sizes[r]
            if draw:
                plan = plan_relation_batches([sizes[r] for r in present], batch_size, self.host_generator)
            else:
                plan = [(gi, off, min(batch_size, sizes[r] - off)) for gi, r in enumerate(present)
                        for off in range(0, sizes[r], batch_size)]
            starts = [begin[present[gi]] + off for gi, off, _ in plan]
            lengths = [ln for _, _, ln in plan]
            rels = [present[gi] for gi, _, _ in plan]
        calls, i = [], 0
        while i < len(starts):
            j = i + 1
            if lengths[i] == batch_size:
                while j < len(starts) and j - i < workers and lengths[j] == batch_size:
                    j += 1
            calls.append((i, j - i, lengths[i]))
            i = j
        return order, starts, rels, calls

    def _call_edges(self, lhs, rhs, rel, starts, rels, first, k, b_now, starts_dev):
        """The [k * b_now] edges of one call and its relation argument."""
        dynamic = self.spec_args["dynamic"]
        if rels is None:  # consecutive batches
            sl = slice(starts[first], starts[first] + k * b_now)
            r = rel[sl].contiguous() if dynamic else rel[sl][::b_now].contiguous()
            return lhs[sl].contiguous(), rhs[sl].contiguous(), r
        idx = (starts_dev[first:first + k, None] + torch.arange(b_now, device=lhs.device)).reshape(-1)
        return lhs[idx], rhs[idx], torch.tensor(rels[first:first + k], dtype=torch.int64, device=lhs.device)

    def _runner(self, runners, tables, k: int, b_now: int, **spec_overrides) -> native.StepRunner:
        runner = runners.get((k, b_now))
        if runner is None:
            (w_l, g_l), (w_r, g_r) = tables[0], tables[-1]
            shared = len(tables) == 1
            spec = native.StepSpec(batch_size=b_now, num_workers=k, **{**self.spec_args, **spec_overrides})
            glob, sums = self.global_embs if self.global_embs is not None else (None, None)
            runner = native.StepRunner(spec, w_l, g_l, None if shared else w_r, None if shared else g_r, *self.ops,
                                       global_embs=glob, global_sums=sums)
            runners[(k, b_now)] = runner
        return runner

    def _uniform(self, k: int, chunks: int, u: int, rows: int, side: int) -> torch.Tensor:
        if self.negatives is not None:
            return self.negatives(k, chunks, u, rows, self.generator, self.device)
        self.calls += 1
        return native.sample_uniform_negatives((self.seed * 0x9E3779B97F4A7C15 + self.calls) & (2**64 - 1), side, rows,
                                               (k, chunks, u), self.device)

    def _evaluate(self, tables, lhs, rhs, rel, eval_idx: torch.Tensor) -> Stats:
        """Ranks the held-out edges (train_cpu.py:886-911, eval.py:43-81) with the
        evaluation-time numbers of negatives; sums, to be averaged by the caller."""
        dev = self.device
        idx = eval_idx.to(dev)
        lhs, rhs, rel = lhs[idx], rhs[idx], rel[idx]
        nb, nu = self.eval_negs
        bsz = round_up_to_nearest_multiple(self.batch_size, nb) if nb > 0 else self.batch_size
        order, starts, rels, calls = self._call_plan(rel, bsz, min(self.num_workers, 8), draw=False)
        if order is not None:
            lhs, rhs, rel = lhs[order], rhs[order], rel[order]
        starts_dev = torch.tensor(starts, dtype=torch.int64, device=dev) if rels is not None else None
        rows_l, rows_r = tables[0][0].shape[0], tables[-1][0].shape[0]
        runners: Dict[Tuple[int, int], native.StepRunner] = {}
        stats = []
        for first, k, b_now in calls:
            runner = self._runner(runners, tables, k, b_now, num_batch_negs=nb, num_uniform_negs=nu)
            l, r, t = self._call_edges(lhs, rhs, rel, starts, rels, first, k, b_now, starts_dev)
            c = runner.spec.num_chunks
            ul = self._uniform(k, c, nu, rows_l, 0) if nu else None
            ur = self._uniform(k, c, nu, rows_r, 1) if nu else None
            count = k * b_now
            # ranks, loss (AbstractBatchProcessor.calc_loss, batching.py:139-150, with relation weights of 1) and the
            # AUC count per edge from one call; the [K, B, N] score tensors are never formed
            self.eval_calls += 1
            _, _, lhs_rank, rhs_rank, loss_edge, hits = runner.ranks(l, r, t, ul, ur, auc_samples=count,
                                                                     auc_seed=(self.seed << 20) + self.eval_calls)
            sides = [s for s, off in ((0, runner.spec.disable_lhs_negs), (1, runner.spec.disable_rhs_negs)) if not off]
            stats.append(ranking_stats_from_ranks([(lhs_rank, rhs_rank)[s] for s in sides], float(loss_edge.sum()), count,
                                                  [hits[s] for s in sides], count))
        return Stats.sum(stats)

    def _train_bucket(self, b: Bucket, tables) -> BucketStats:
        dev = self.device
        lhs, rhs, rel = (t.to(dev, non_blocking=True) for t in self.edges[b])
        n = lhs.shape[0]
        if n == 0:
            return BucketStats(b, 0, 0.0, 0, 0)
        eval_idx = holdout_indices(n, self.eval_fraction, b)
        eval_before = self._evaluate(tables, lhs, rhs, rel, eval_idx) if eval_idx is not None else None
        num_train = n - (eval_idx.shape[0] if eval_idx is not None else 0)
        if self.edge_order is not None:
            perm = self.edge_order(b, num_train).to(dev)
        else:  # _coordinate_train shuffles the bucket's training edges (train_cpu.py:857-859)
            perm = native.randperm(num_train, hash((self.seed, self.epoch, b.lhs, b.rhs)) & 0x7FFFFFFF, dev)
        if eval_idx is not None:
            perm = train_edge_indices(n, eval_idx, dev)[perm]
        lhs_t, rhs_t, rel_t = lhs[perm], rhs[perm], rel[perm]
        order, starts, rels, calls = self._call_plan(rel_t, self.batch_size, self.num_workers, draw=True)
        if order is not None:
            lhs_t, rhs_t, rel_t = lhs_t[order], rhs_t[order], rel_t[order]
        starts_dev = torch.tensor(starts, dtype=torch.int64, device=dev) if rels is not None else None
        rows_l, rows_r = tables[0][0].shape[0], tables[-1][0].shape[0]
        u = self.spec_args["num_uniform_negs"]
        # every call leaves its batches' statistics in its own row; one reduction per bucket
        k_max = max((k for _, k, _ in calls), default=1)
        loss_all = torch.zeros((len(calls), k_max), dtype=torch.float32, device=dev)
        viol_all = torch.zeros((len(calls), k_max, 2), dtype=torch.int64, device=dev)
        runners: Dict[Tuple[int, int], native.StepRunner] = {}
        for i, (first, k, b_now) in enumerate(calls):
            runner = self._runner(runners, tables, k, b_now)
            stats_out = (loss_all[i, :k], viol_all[i, :k])
            l, r, t = self._call_edges(lhs_t, rhs_t, rel_t, starts, rels, first, k, b_now, starts_dev)
            if self.calls_log is not None:
                self.calls_log.append(dict(bucket=b, epoch=self.epoch, workers=k, batch_size=b_now, lhs=l.cpu(),
                                           rhs=r.cpu(), rel=t.cpu()))
            c = runner.spec.num_chunks
            if u and self.negatives is not None:
                runner.train(l, r, t, self._uniform(k, c, u, rows_l, 0), self._uniform(k, c, u, rows_r, 1), stats_out=stats_out)
            else:
                self.calls += 1
                call_seed = (self.seed * 0x9E3779B97F4A7C15 + self.calls) & (2**64 - 1) if u else None
                runner.train(l, r, t, uniform_seed=call_seed, stats_out=stats_out)
        eval_after = self._evaluate(tables, lhs, rhs, rel, eval_idx) if eval_idx is not None else None
        loss = float(loss_all.double().sum())
        v = viol_all.sum(dim=(0, 1)).tolist()
        return BucketStats(b, num_train, loss, int(v[0]), int(v[1]), eval_before, eval_after)

    def train_epoch(self) -> List[BucketStats]:
        buckets = [b for b in create_ordered_buckets(self.nparts_lhs, self.nparts_rhs, self.bucket_order,
                                                     generator=self.rng) if b in self.edges]
        stats = []
        for i, b in enumerate(buckets):
            keys = self._keys(b)
            tables = self.cache.acquire(keys)
            if i + 1 < len(buckets):  # the next bucket's partitions travel while this one trains
                self.cache.prefetch(self._keys(buckets[i + 1]), keys)
            else:
                self.cache.write_back_idle(keys)
            stats.append(self._train_bucket(b, tables))
            self.cache.release(keys)
        self.cache.flush()
        self.epoch += 1
        return stats

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
(batching.py:109-112).
"""
import random
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from . import native

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
            self._write_back(slot)
            del self.by_key[slot.key]
        n = self.store.rows(key)
        with torch.cuda.stream(self.copy_stream):
            # a buffer taken over from another partition: its write-back precedes this upload on the same stream
            slot.w[:n].copy_(self.store.tables[key], non_blocking=True)
            slot.g[:n].copy_(self.store.sums[key], non_blocking=True)
            slot.ready = torch.cuda.Event()
            slot.ready.record(self.copy_stream)
        slot.key, slot.last_use = key, None
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
            slot.last_use = torch.cuda.Event()
            slot.last_use.record(torch.cuda.current_stream(self.device))

    def flush(self) -> None:
        """Writes every resident partition back to the store and waits for it."""
        for slot in self.slots:
            if slot.key is not None:
                self._write_back(slot)
        self.copy_stream.synchronize()


@dataclass
class BucketStats:
    bucket: Bucket
    num_edges: int
    loss: float
    violators_lhs: int
    violators_rhs: int


class BucketLoop:
    """One pass over all buckets = ``train_epoch()``.

    edges: {Bucket: (lhs, rhs, rel)} int64 tensors of partition-local offsets and
    relation types, on the host (pinned or not) or already on the device.
    Standard (non-dynamic) relations need single-relation batches: pass one
    relation type overall or dynamic=True.
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
                 edge_order: Optional[Callable[[Bucket, int], torch.Tensor]] = None,
                 negatives: Optional[Callable[..., torch.Tensor]] = None) -> None:
        self.store, self.edges = store, edges
        self.lhs_entity, self.rhs_entity = lhs_entity, rhs_entity
        self.nparts_lhs, self.nparts_rhs = nparts_lhs, nparts_rhs
        self.device = torch.device(device)
        self.batch_size, self.num_workers = batch_size, num_workers
        self.spec_args = dict(dim=dim, num_batch_negs=num_batch_negs, num_uniform_negs=num_uniform_negs,
                              operator=operator, dynamic=dynamic, num_relations=num_relations, comparator=comparator,
                              loss=loss, margin=margin, lr=lr, relation_lr=relation_lr)
        self.ops = (rhs_op or {}, rhs_op_sum or {}, lhs_op or {}, lhs_op_sum or {})
        self.cache = PartitionCache(store, self.device, resident_partitions)
        self.bucket_order = bucket_order
        self.rng = random.Random(seed)
        self.generator = torch.Generator(device=self.device).manual_seed(seed)
        self.seed = seed
        self.edge_order = edge_order
        # None: the step draws its uniform negatives itself (SimpleEmbedding.sample_entities,
        # model.py:70-75), one seed per call; a callable(workers, chunks, num_uniform, num_rows,
        # generator, device) -> [workers, chunks, num_uniform] supplies them instead
        self.negatives = negatives
        self.calls = 0
        self.epoch = 0

    def _keys(self, b: Bucket) -> List[PartitionKey]:
        keys = [(self.lhs_entity, b.lhs)]
        if (self.rhs_entity, b.rhs) != keys[0]:
            keys.append((self.rhs_entity, b.rhs))
        return keys

    def _train_bucket(self, b: Bucket, tables) -> BucketStats:
        dev = self.device
        lhs, rhs, rel = (t.to(dev, non_blocking=True) for t in self.edges[b])
        n = lhs.shape[0]
        if n == 0:
            return BucketStats(b, 0, 0.0, 0, 0)
        if self.edge_order is not None:
            perm = self.edge_order(b, n).to(dev)
        else:  # _coordinate_train shuffles the bucket's edges (train_cpu.py:857-859)
            perm = native.randperm(n, hash((self.seed, self.epoch, b.lhs, b.rhs)) & 0x7FFFFFFF, dev)
        lhs, rhs, rel = lhs[perm], rhs[perm], rel[perm]
        (w_l, g_l) = tables[0]
        (w_r, g_r) = tables[-1]
        shared = len(tables) == 1
        dynamic = self.spec_args["dynamic"]
        bsz, kmax = self.batch_size, self.num_workers
        u = self.spec_args["num_uniform_negs"]
        if not dynamic and self.spec_args["num_relations"] != 1:
            raise NotImplementedError("standard (non-dynamic) relations need single-relation batches: "
                                      "use one relation type or dynamic=True")
        loss = torch.zeros((), dtype=torch.float64, device=dev)
        viol = torch.zeros(2, dtype=torch.int64, device=dev)
        runners: Dict[Tuple[int, int], native.StepRunner] = {}
        off = 0
        while off < n:
            left = n - off
            if left >= bsz:
                k, b_now = min(kmax, left // bsz), bsz
            else:
                k, b_now = 1, left  # the final partial batch (batching.py:109-112)
            runner = runners.get((k, b_now))
            if runner is None:
                spec = native.StepSpec(batch_size=b_now, num_workers=k, **self.spec_args)
                runner = native.StepRunner(spec, w_l, g_l, None if shared else w_r, None if shared else g_r, *self.ops)
                runners[(k, b_now)] = runner
            spec = runner.spec
            count = k * b_now
            sl = slice(off, off + count)
            if dynamic:
                r = rel[sl].contiguous()
            else:
                r = rel[off:off + count:b_now].contiguous()  # one relation type per batch
            c = spec.num_chunks
            if u and self.negatives is not None:
                ul = self.negatives(k, c, u, w_l.shape[0], self.generator, dev)
                ur = self.negatives(k, c, u, w_r.shape[0], self.generator, dev)
                runner.train(lhs[sl].contiguous(), rhs[sl].contiguous(), r, ul, ur)
            else:
                self.calls += 1
                call_seed = (self.seed * 0x9E3779B97F4A7C15 + self.calls) & (2**64 - 1) if u else None
                runner.train(lhs[sl].contiguous(), rhs[sl].contiguous(), r, uniform_seed=call_seed)
            loss += runner.loss_out.double().sum()
            viol += runner.violators_out.sum(dim=0)
            off += count
        v = viol.tolist()
        return BucketStats(b, n, float(loss), int(v[0]), int(v[1]))

    def train_epoch(self) -> List[BucketStats]:
        buckets = [b for b in create_ordered_buckets(self.nparts_lhs, self.nparts_rhs, self.bucket_order,
                                                     generator=self.rng) if b in self.edges]
        stats = []
        for i, b in enumerate(buckets):
            keys = self._keys(b)
            tables = self.cache.acquire(keys)
            if i + 1 < len(buckets):  # the next bucket's partitions travel while this one trains
                self.cache.prefetch(self._keys(buckets[i + 1]), keys)
            stats.append(self._train_bucket(b, tables))
            self.cache.release(keys)
        self.cache.flush()
        self.epoch += 1
        return stats

"""The reference's HOGWILD training loop, restated over ``oracle.step`` (test
infrastructure / CPU baseline only; bench.py times it, nothing ships it).

Follows train_cpu.py:849-884 (_coordinate_train: a random edge permutation is
split almost equally among `workers` pool processes) and util.py:281-314
(spawn pool, every worker single-threaded and seeded from its pid, tables in
shared memory, no locks); each worker runs batching.py:91-125 over its slice:
contiguous batches, uniform negatives drawn by torch.randint inside the step
(model.py:70-75), Trainer._process_one_batch per batch.
"""
import os
import time
from typing import Dict, Optional, Tuple

import torch
import torch.multiprocessing as mp

from . import step as ostep


def _worker(rank: int, cfg, shared: Dict[str, torch.Tensor], lhs, rhs, rel, batch_size: int, max_seconds: float,
            barrier, out_queue) -> None:
    # CPU workers must never open the GPU (autograd's first backward() would
    # otherwise ask the HIP runtime for its device count)
    os.environ["HIP_VISIBLE_DEVICES"] = ""
    os.environ["ROCR_VISIBLE_DEVICES"] = ""
    torch.set_num_threads(1)
    torch.manual_seed(os.getpid())
    st = ostep.TrainState(
        w_lhs=shared["w_lhs"], g_lhs=shared["g_lhs"],
        w_rhs=shared.get("w_rhs", shared["w_lhs"]), g_rhs=shared.get("g_rhs", shared["g_lhs"]),
    )
    if "w_rhs" not in shared:
        st.w_rhs, st.g_rhs = st.w_lhs, st.g_lhs
    st.rhs_op = {k[len("rhs_op."):]: v for k, v in shared.items() if k.startswith("rhs_op.")}
    st.rhs_op_sum = {k[len("rhs_sum."):]: v for k, v in shared.items() if k.startswith("rhs_sum.")}
    st.lhs_op = {k[len("lhs_op."):]: v for k, v in shared.items() if k.startswith("lhs_op.")}
    st.lhs_op_sum = {k[len("lhs_sum."):]: v for k, v in shared.items() if k.startswith("lhs_sum.")}
    n = lhs.shape[0]
    n_l, n_r = st.w_lhs.shape[0], st.w_rhs.shape[0]
    u = cfg.num_uniform_negs

    def one_batch(off: int) -> int:
        bl, br = lhs[off:off + batch_size], rhs[off:off + batch_size]
        if cfg.dynamic:
            brel = rel[off:off + batch_size]
        else:
            brel = int(rel[off])
        _, c, _ = cfg.chunking(bl.shape[0])
        ul = torch.randint(0, n_l, (c, u)) if u > 0 else None
        ur = torch.randint(0, n_r, (c, u)) if u > 0 else None
        ostep.train_step(cfg, st, bl, br, brel, ul, ur)
        return bl.shape[0]

    one_batch(0)  # warm-up: first-touch of the op kernels
    barrier.wait()
    t0 = time.perf_counter()
    done, off = 0, 0
    while time.perf_counter() - t0 < max_seconds:
        if off + batch_size > n:
            off = 0
        done += one_batch(off)
        off += batch_size
    out_queue.put((rank, done, time.perf_counter() - t0))


def run(cfg, w_lhs: torch.Tensor, lhs: torch.Tensor, rhs: torch.Tensor, rel: torch.Tensor, batch_size: int,
        workers: int, max_seconds: float, w_rhs: Optional[torch.Tensor] = None) -> Tuple[float, int, float]:
    """Trains for about `max_seconds` with `workers` HOGWILD processes on a copy
    of the tables; returns (edges_per_second, edges_trained, wall_seconds).
    In standard mode `rel` must be constant inside every batch-sized slice."""
    st = ostep.make_state(cfg, w_lhs.clone(), None if w_rhs is None else w_rhs.clone())
    shared = {"w_lhs": st.w_lhs, "g_lhs": st.g_lhs}
    if w_rhs is not None:
        shared["w_rhs"], shared["g_rhs"] = st.w_rhs, st.g_rhs
    for prefix, d in (("rhs_op.", st.rhs_op), ("rhs_sum.", st.rhs_op_sum), ("lhs_op.", st.lhs_op), ("lhs_sum.", st.lhs_op_sum)):
        for k, v in d.items():
            shared[prefix + k] = v
    for v in shared.values():
        v.share_memory_()
    ctx = mp.get_context("spawn")
    barrier = ctx.Barrier(workers)
    queue = ctx.Queue()
    perm = torch.randperm(lhs.shape[0])
    # split_almost_equally (util.py:227-236)
    per = lhs.shape[0] // workers + (1 if lhs.shape[0] % workers else 0)
    procs = []
    saved_env = {k: os.environ.get(k) for k in ("HIP_VISIBLE_DEVICES", "ROCR_VISIBLE_DEVICES")}
    os.environ["HIP_VISIBLE_DEVICES"] = ""
    os.environ["ROCR_VISIBLE_DEVICES"] = ""
    for r in range(workers):
        sl = perm[min(r * per, lhs.shape[0]):min((r + 1) * per, lhs.shape[0])]
        if not cfg.dynamic:
            sl = sl.sort().values  # keep batch-sized slices single-relation when edges are grouped by relation
        p = ctx.Process(target=_worker, args=(r, cfg, shared, lhs[sl].clone(), rhs[sl].clone(), rel[sl].clone(),
                                              batch_size, max_seconds, barrier, queue))
        p.start()
        procs.append(p)
    for k, v in saved_env.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v
    # fail fast when a worker dies (util.py:320-347 polls the same way)
    import queue as queue_mod

    results = []
    while len(results) < workers:
        try:
            results.append(queue.get(timeout=1.0))
        except queue_mod.Empty:
            dead = [p for p in procs if p.exitcode not in (None, 0)]
            if dead:
                for p in procs:
                    if p.is_alive():
                        p.terminate()
                raise RuntimeError(f"{len(dead)} HOGWILD worker(s) exited with an error")
    for p in procs:
        p.join()
    edges = sum(r[1] for r in results)
    wall = max(r[2] for r in results)
    return edges / wall, edges, wall

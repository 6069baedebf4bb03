"""numpy restatement of the reference's native helpers (test infrastructure only).

Follows torchbiggraph/util.cpp: reversePermutation :104-125, shuffle :127-220,
subBucket :260-423, and the *contract* of randperm :14-102 (its exact output
depends on the thread count and on at::CPUGeneratorImpl, so only "is a uniform
random permutation" is portable).
"""
from typing import Dict, List, Sequence, Tuple

import numpy as np


def reverse_permutation(perm: np.ndarray) -> np.ndarray:
    """res[perm[i]] = i  (util.cpp:110-113)."""
    perm = np.asarray(perm, dtype=np.int64)
    res = np.empty_like(perm)
    for i in range(perm.shape[0]):
        res[perm[i]] = i
    return res


def shuffle(rows: np.ndarray, perm: np.ndarray) -> np.ndarray:
    """Returns what the in-place cycle walk of util.cpp:177-207 leaves behind:
    the row that was at i ends up at perm[i]."""
    perm = np.asarray(perm, dtype=np.int64)
    if perm.ndim != 1:
        raise ValueError("Permutation must have exactly one dimension")
    if rows.ndim < 1:
        raise ValueError("Tensor must have at least one dimension")
    if rows.shape[0] != perm.shape[0]:
        raise ValueError(
            "Tensor and permutation must have the same number of elements on the first dimension"
        )
    if perm.size and (perm.min() < 0 or perm.max() >= perm.shape[0]):
        raise ValueError("Permutation has out-of-bound values")
    out = rows.copy()
    done = np.zeros(perm.shape[0], dtype=bool)
    for base in range(perm.shape[0]):
        if done[base]:
            continue
        carried = rows[base].copy()
        done[base] = True
        cur = base
        while True:
            cur = int(perm[cur])
            nxt = rows[cur].copy()
            finished = bool(done[cur])
            done[cur] = True
            out[cur] = carried
            carried = nxt
            if finished:
                break
    return out


def sub_bucket(
    lhs_in: np.ndarray,
    rhs_in: np.ndarray,
    rel_in: np.ndarray,
    lhs_entity_counts: Sequence[int],
    lhs_perms: Sequence[np.ndarray],
    rhs_entity_counts: Sequence[int],
    rhs_perms: Sequence[np.ndarray],
    num_lhs_sub_parts: int,
    num_rhs_sub_parts: int,
    dynamic_relations: bool,
) -> Tuple[np.ndarray, np.ndarray, np.ndarray, Dict[Tuple[int, int], Tuple[int, int]]]:
    """(lhs_out, rhs_out, rel_out, {(i, j): (start, stop)}) as util.cpp:260-423:
    edges keep their input order inside each sub-bucket (thread ranges are
    ascending, so the result does not depend on the thread count)."""
    n = rel_in.shape[0]
    num_rel = len(lhs_perms)
    if len(rhs_perms) != num_rel or len(lhs_entity_counts) != num_rel or len(rhs_entity_counts) != num_rel:
        raise RuntimeError("Inconsistent num_relations")

    def part_size(count: int, parts: int) -> int:
        return count // parts + (1 if count % parts != 0 else 0)

    lhs_sizes = [part_size(c, num_lhs_sub_parts) for c in lhs_entity_counts]
    rhs_sizes = [part_size(c, num_rhs_sub_parts) for c in rhs_entity_counts]
    buckets: List[List[Tuple[int, int, int]]] = [
        [] for _ in range(num_lhs_sub_parts * num_rhs_sub_parts)
    ]
    for e in range(n):
        r = 0 if dynamic_relations else int(rel_in[e])
        if r >= num_rel:
            raise RuntimeError("rel > numRelations")
        lo = int(lhs_perms[r][lhs_in[e]])
        ro = int(rhs_perms[r][rhs_in[e]])
        b = (lo // lhs_sizes[r]) * num_rhs_sub_parts + ro // rhs_sizes[r]
        buckets[b].append((lo % lhs_sizes[r], ro % rhs_sizes[r], int(rel_in[e])))
    lhs_out = np.empty(n, dtype=np.int64)
    rhs_out = np.empty(n, dtype=np.int64)
    rel_out = np.empty(n, dtype=np.int64)
    ranges: Dict[Tuple[int, int], Tuple[int, int]] = {}
    off = 0
    for i in range(num_lhs_sub_parts):
        for j in range(num_rhs_sub_parts):
            items = buckets[i * num_rhs_sub_parts + j]
            ranges[(i, j)] = (off, off + len(items))
            for (a, b_, c) in items:
                lhs_out[off], rhs_out[off], rel_out[off] = a, b_, c
                off += 1
    return lhs_out, rhs_out, rel_out, ranges


def is_permutation(perm: np.ndarray) -> bool:
    perm = np.asarray(perm)
    n = perm.shape[0]
    if n == 0:
        return True
    if perm.min() < 0 or perm.max() >= n:
        return False
    return bool(np.bincount(perm, minlength=n).max() == 1)

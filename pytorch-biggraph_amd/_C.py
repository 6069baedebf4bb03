"""GPU versions of the reference's `_C` extension module (reference:
torchbiggraph/util.cpp:425-460): same function names, argument order and error
behaviour; tensors live on the GPU and `num_threads` is accepted and ignored."""
from typing import Dict, List, Sequence, Tuple

import torch

from . import native

# at::default_rng_seed_val, which the reference hands to every thread when seed < 0
_DEFAULT_SEED = 67280421310721


def randperm(num_items: int, num_threads: int = 1, seed: int = -1, device="cuda") -> torch.Tensor:
    """A uniform random permutation of range(num_items) (util.cpp:14-102).  The
    reference's bit pattern depends on its thread count; only the contract is kept."""
    return native.randperm(int(num_items), _DEFAULT_SEED if seed < 0 else int(seed), torch.device(device))


def reverse_permutation(perm: torch.Tensor, num_threads: int = 1) -> torch.Tensor:
    """res[perm[i]] = i (util.cpp:104-125)."""
    return native.reverse_permutation(perm.contiguous())


def shuffle(tensor: torch.Tensor, permutation: torch.Tensor, num_threads: int = 1) -> None:
    """In place: the row at i moves to permutation[i] (util.cpp:127-220)."""
    if permutation.dtype != torch.int64:
        raise ValueError("Permutation must have int64 dtype")
    if permutation.dim() != 1:
        raise ValueError("Permutation must have exactly one dimension")
    if tensor.dim() < 1:
        raise ValueError("Tensor must have at least one dimension")
    num_rows = tensor.shape[0]
    if num_rows != permutation.shape[0]:
        raise ValueError("Tensor and permutation must have the same number of elements on the first dimension")
    if num_rows == 0:
        return
    if tensor.stride(0) == 0:
        return
    if not tensor[0].is_contiguous():
        raise ValueError("Each sub-tensor of tensor (along the first dimension) must be contiguous")
    for i in range(1, tensor.dim()):
        if tensor.stride(i) == 0:
            raise ValueError("Tensor cannot have strides that are zero (for now)")
    if tensor.stride(0) != tensor[0].numel():
        raise ValueError("Rows must be densely packed")
    native.shuffle_rows(tensor, permutation.contiguous())


def sub_bucket(
    lhs_in: torch.Tensor, rhs_in: torch.Tensor, rel_in: torch.Tensor,
    lhs_entity_counts: Sequence[int], lhs_perms: Sequence[torch.Tensor],
    rhs_entity_count: Sequence[int], rhs_perms: Sequence[torch.Tensor],
    lhs_out: torch.Tensor, rhs_out: torch.Tensor, rel_out: torch.Tensor,
    num_lhs_sub_parts: int, num_rhs_sub_parts: int, num_threads: int = 1, dynamic_relations: bool = False,
) -> Dict[Tuple[int, int], Tuple[torch.Tensor, torch.Tensor, torch.Tensor]]:
    """Splits a bucket's edges into num_lhs_sub_parts x num_rhs_sub_parts
    sub-buckets, keeping the input order inside each (util.cpp:260-423).  The
    returned tensors are views of lhs_out / rhs_out / rel_out."""
    num_rel = len(lhs_perms)
    if len(rhs_perms) != num_rel or len(lhs_entity_counts) != num_rel or len(rhs_entity_count) != num_rel:
        raise RuntimeError("Inconsistent num_relations")

    def part_sizes(counts: Sequence[int], parts: int) -> List[int]:
        return [c // parts + (1 if c % parts != 0 else 0) for c in counts]

    offsets = native.sub_bucket(
        lhs_in, rhs_in, rel_in, lhs_perms, rhs_perms, part_sizes(lhs_entity_counts, num_lhs_sub_parts),
        part_sizes(rhs_entity_count, num_rhs_sub_parts), num_lhs_sub_parts, num_rhs_sub_parts, dynamic_relations,
        lhs_out, rhs_out, rel_out).tolist()
    res = {}
    for i in range(num_lhs_sub_parts):
        for j in range(num_rhs_sub_parts):
            a, b = offsets[i * num_rhs_sub_parts + j], offsets[i * num_rhs_sub_parts + j + 1]
            res[(i, j)] = (lhs_out[a:b], rhs_out[a:b], rel_out[a:b])
    return res

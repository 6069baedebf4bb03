"""Host-side helpers of the step (reference: torchbiggraph/util.py:42-118,
227-244, 260-278)."""
from typing import Any, Callable, Dict, Iterable, List, Mapping, Optional, Tuple, Union

import torch
from torch.optim import Optimizer


def match_shape(tensor: torch.Tensor, *expected_shape: Union[int, type(Ellipsis)]) -> Union[None, int, Tuple[int, ...]]:
    """Checks `tensor`'s shape against a pattern of ints, -1 (any size, returned)
    and at most one Ellipsis (any number of dimensions); TypeError on mismatch
    (reference: util.py:42-118)."""
    for d in expected_shape:
        if not (isinstance(d, int) or d is Ellipsis):
            raise RuntimeError("Some arguments aren't ints or ellipses: %s" % (expected_shape,))
    actual = tuple(tensor.size())

    def mismatch() -> TypeError:
        want = ", ".join("..." if d is Ellipsis else "*" if d < 0 else "%d" % d for d in expected_shape)
        return TypeError("Shape doesn't match: (%s) != (%s)" % (", ".join("%d" % d for d in actual), want))

    n_ellipsis = sum(1 for d in expected_shape if d is Ellipsis)
    if n_ellipsis > 1:
        raise RuntimeError("Two or more ellipses in %s" % (tuple(expected_shape),))
    if n_ellipsis == 0:
        if len(actual) != len(expected_shape):
            raise mismatch()
        pattern = list(expected_shape)
    else:
        fixed = len(expected_shape) - 1
        if len(actual) < fixed:
            raise mismatch()
        at = expected_shape.index(Ellipsis)
        tail = fixed - at
        middle = list(actual[at:len(actual) - tail])
        pattern = list(expected_shape[:at]) + middle + list(expected_shape[at + 1:])
    unknown: List[int] = []
    for have, want in zip(actual, pattern):
        if want < 0:
            unknown.append(have)
        elif have != want:
            raise mismatch()
    if not unknown:
        return None
    if len(unknown) == 1:
        return unknown[0]
    return tuple(unknown)


def split_almost_equally(size: int, *, num_parts: int) -> Iterable[slice]:
    """`num_parts` consecutive slices of ceil(size / num_parts) elements, the
    later ones possibly shorter or empty (reference: util.py:227-236)."""
    step = -(-size // num_parts)
    for i in range(num_parts):
        yield slice(min(i * step, size), min((i + 1) * step, size))


def div_roundup(num: int, denom: int) -> int:
    return (num + denom - 1) // denom


def round_up_to_nearest_multiple(value: int, factor: int) -> int:
    return ((value - 1) // factor + 1) * factor


class DummyOptimizer(Optimizer):
    """Optimizer over no parameters (reference: util.py:260-278)."""

    def __init__(self) -> None:
        super().__init__([{"params": []}], {})

    def step(self, closure: Optional[Callable[[], torch.Tensor]] = None) -> None:
        pass

    def state_dict(self) -> Dict[str, Any]:
        return {}

    def load_state_dict(self, state_dict: Mapping[str, Any]) -> None:
        pass

    def share_memory(self) -> None:
        pass

"""Name-keyed plugin registries (reference: torchbiggraph/plugin.py:16-40).

The package keeps registries of its own under the reference's names: operators
``none | diagonal | translation | linear | affine | complex_diagonal``, comparators
``dot | cos | l2 | squared_l2``, loss functions ``ranking | logistic | softmax``
and the regularizer ``N3``.
"""
from typing import Callable, Dict, Generic, Type, TypeVar

T = TypeVar("T")


class PluginRegistry(Generic[T]):
    def __init__(self) -> None:
        self.registry: Dict[str, Type[T]] = {}

    def register(self, name: str, class_: Type[T]) -> None:
        existing = self.registry.get(name)
        if existing is None:
            self.registry[name] = class_
        elif existing is not class_:
            raise RuntimeError(f"Attempting to re-register {name} which was already set to {existing!r}")

    def register_as(self, name: str) -> Callable[[Type[T]], Type[T]]:
        def decorator(class_: Type[T]) -> Type[T]:
            self.register(name, class_)
            return class_

        return decorator

    def get_class(self, name: str) -> Type[T]:
        if name not in self.registry:
            known = ", ".join(sorted(self.registry))
            raise NotImplementedError(f"Unknown name {name} (known names: {known})")
        return self.registry[name]

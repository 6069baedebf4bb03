"""MI355X-native implementation of PyTorch-BigGraph's per-bucket training step.

Import name: ``pytorch_biggraph_amd`` (the directory is ``pytorch-biggraph_amd``;
``__graft_entry__.load_package()`` registers it under the importable name).

The modules mirror the reference's interface for the path: ``plugin``
(registries), ``operators``, ``model`` (embeddings, comparators,
MultiRelationEmbedder), ``losses``, ``regularizers``, ``row_adagrad``, ``async_adagrad``,
``batching``, ``train`` (Trainer), ``bucket_loop`` (partition swap and the per-bucket loop), ``eval`` (RankingEvaluator), ``_C`` (permutation helpers), ``edgelist`` /
``entitylist`` / ``stats`` / ``types`` / ``util`` / ``config``.  ``native`` holds
the tensor-level wrappers over the C ABI and ``_lib`` the ctypes binding.
"""
from . import _lib, native  # noqa: F401
from .native import StepRunner, StepSpec  # noqa: F401
from . import (  # noqa: F401
    _C, async_adagrad, batching, bucket_loop, config, edgelist, entitylist, eval, losses, model, operators, plugin, regularizers, row_adagrad, stats,
    train, types, util,
)

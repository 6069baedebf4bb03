"""CPU oracle for the PyTorch-BigGraph per-bucket training step.

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, on the
CPU, the algorithm of the reference's training step so that the HIP kernels
can be checked against it.  Only ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py`` may import it; the shipped package
never does, and never falls back to it.

Modules
-------
``step``      gather -> operator -> comparator.prepare -> chunked negatives ->
              scores -> masks -> loss -> backward -> RowAdagrad / AsyncAdagrad,
              written with torch CPU tensor ops in the reference's own order of
              operations (reference: torchbiggraph/model.py:478-856,
              operators.py:49-338, losses.py:53-161, batching.py:139-150,
              train_cpu.py:86-112, row_adagrad.py:80-107,
              async_adagrad.py:51-85).
``brute``     an independent float64 per-edge restatement of the scoring and
              masking rules (no chunk tensors, no bmm), used to pin ``step``.
``perm``      numpy restatement of torchbiggraph/util.cpp:14-423
              (randperm contract, reverse_permutation, shuffle, sub_bucket).
``hogwild``   the multi-process HOGWILD loop of train_cpu.py:849-884 over
              ``step``; it is what ``bench.py`` times as the CPU baseline.

Parity pinning (what each function is checked against before it is trusted):
operators, comparators, gather and losses replay every literal vector of the
reference's test/test_model.py and test/test_losses.py (tests/golden/*.json);
the chunk/mask logic is pinned by ``brute`` and by closed-form invariants
(all_negs also by its equality with uniform-only negatives over every entity,
the bias inside the step also by its reduction to the base comparator and by
the shift of all scores under a shift of all biases; the N3 regularizer by
numpy complex arithmetic, closed forms and central differences; the global
embeddings by the shifted-table identity);
RowAdagrad by its reduction to torch.optim.Adagrad on constant-row gradients
and on dim 1, and by pre-summed duplicates; AsyncAdagrad by torch.optim.Adagrad;
reverse_permutation / shuffle / sub_bucket by the reference's own util.cpp
compiled into oracle/_ref (when built) and by argsort / index_copy / stable
sort identities; half_precision (no vector in the reference's tests, and its cast
only happens on a CUDA device) by the fp32 path on inputs whose intermediates are
all float16 numbers and by a numpy float16 restatement of every rounding point
(tests/test_oracle_half.py).  randperm's bit pattern is not portable (it depends on the
thread count): only its contract (a uniform random permutation) is checked,
so its bits are "parity unpinned" by design.
"""

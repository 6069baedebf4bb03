"""oracle.perm against the reference's own util.cpp (compiled into oracle/_ref)
and against identities that fix the semantics without it."""
import numpy as np
import pytest
import torch

from oracle import perm as operm


def rand_perm(n, seed):
    return np.random.default_rng(seed).permutation(n).astype(np.int64)


@pytest.mark.parametrize("n", [0, 1, 2, 17, 1000])
def test_reverse_permutation_identities(n):
    p = rand_perm(n, n)
    r = operm.reverse_permutation(p)
    assert np.array_equal(r, np.argsort(p))
    assert np.array_equal(r[p], np.arange(n))


@pytest.mark.parametrize("n,width", [(0, 3), (1, 1), (7, 5), (500, 4)])
def test_shuffle_is_scatter_by_perm(n, width):
    p = rand_perm(n, n + 1)
    rows = np.random.default_rng(0).standard_normal((n, width)).astype(np.float32)
    out = operm.shuffle(rows, p)
    want = np.empty_like(rows)
    want[p] = rows
    assert np.array_equal(out, want)
    # the reverse permutation undoes it
    assert np.array_equal(operm.shuffle(out, operm.reverse_permutation(p)), rows)


def test_shuffle_errors():
    with pytest.raises(ValueError):
        operm.shuffle(np.zeros((3, 2)), np.array([0, 1], dtype=np.int64))
    with pytest.raises(ValueError):
        operm.shuffle(np.zeros((3, 2)), np.array([0, 1, 3], dtype=np.int64))
    with pytest.raises(ValueError):
        operm.shuffle(np.zeros((2, 2)), np.zeros((2, 1), dtype=np.int64))


def sub_bucket_inputs(n_edges, n_rel, seed, dynamic):
    rng = np.random.default_rng(seed)
    counts_l = [int(c) for c in rng.integers(5, 40, n_rel)]
    counts_r = [int(c) for c in rng.integers(5, 40, n_rel)]
    rel = rng.integers(0, n_rel, n_edges).astype(np.int64)
    look = np.zeros(n_edges, dtype=np.int64) if dynamic else rel
    lhs = np.array([rng.integers(0, counts_l[r]) for r in look], dtype=np.int64).reshape(n_edges)
    rhs = np.array([rng.integers(0, counts_r[r]) for r in look], dtype=np.int64).reshape(n_edges)
    perms_l = [rng.permutation(c).astype(np.int64) for c in counts_l]
    perms_r = [rng.permutation(c).astype(np.int64) for c in counts_r]
    return lhs, rhs, rel, counts_l, perms_l, counts_r, perms_r


@pytest.mark.parametrize("dynamic", [False, True])
@pytest.mark.parametrize("parts", [(1, 1), (2, 3), (4, 4)])
def test_sub_bucket_is_a_stable_partition(dynamic, parts):
    lhs, rhs, rel, cl, pl, cr, pr = sub_bucket_inputs(300, 3, 11, dynamic)
    lo, ro, relo, ranges = operm.sub_bucket(lhs, rhs, rel, cl, pl, cr, pr, parts[0], parts[1], dynamic)
    look = np.zeros_like(rel) if dynamic else rel
    size_l = np.array([-(-c // parts[0]) for c in cl])[look]
    size_r = np.array([-(-c // parts[1]) for c in cr])[look]
    off_l = np.array([pl[r][x] for r, x in zip(look, lhs)])
    off_r = np.array([pr[r][x] for r, x in zip(look, rhs)])
    key = (off_l // size_l) * parts[1] + off_r // size_r
    order = np.argsort(key, kind="stable")
    assert np.array_equal(lo, (off_l % size_l)[order])
    assert np.array_equal(ro, (off_r % size_r)[order])
    assert np.array_equal(relo, rel[order])
    counts = np.bincount(key, minlength=parts[0] * parts[1])
    ends = np.cumsum(counts)
    for i in range(parts[0]):
        for j in range(parts[1]):
            b = i * parts[1] + j
            assert ranges[(i, j)] == (int(ends[b] - counts[b]), int(ends[b]))


@pytest.mark.parametrize("threads", [1, 3])
def test_against_reference_util_cpp(ref_C, threads):
    n = 2000
    p = rand_perm(n, 5)
    tp = torch.from_numpy(p)
    assert np.array_equal(ref_C.reverse_permutation(tp, threads).numpy(), operm.reverse_permutation(p))
    for shape, dtype in (((n, 7), torch.float32), ((n,), torch.float32), ((n,), torch.int64), ((n, 2, 3), torch.float64)):
        t = (torch.randn(shape) * 100).to(dtype)
        want = operm.shuffle(t.numpy(), p)
        ref_C.shuffle(t, tp, threads)
        assert np.array_equal(t.numpy(), want)
    for dynamic in (False, True):
        lhs, rhs, rel, cl, pl, cr, pr = sub_bucket_inputs(n, 4, 3, dynamic)
        outs = [torch.empty(n, dtype=torch.int64) for _ in range(3)]
        res = ref_C.sub_bucket(
            torch.from_numpy(lhs), torch.from_numpy(rhs), torch.from_numpy(rel),
            cl, [torch.from_numpy(x) for x in pl], cr, [torch.from_numpy(x) for x in pr],
            outs[0], outs[1], outs[2], 3, 2, threads, dynamic)
        lo, ro, relo, ranges = operm.sub_bucket(lhs, rhs, rel, cl, pl, cr, pr, 3, 2, dynamic)
        assert np.array_equal(outs[0].numpy(), lo)
        assert np.array_equal(outs[1].numpy(), ro)
        assert np.array_equal(outs[2].numpy(), relo)
        for key, (a, b) in ranges.items():
            got = res[key]
            assert got[0].shape[0] == b - a
            assert np.array_equal(got[0].numpy(), lo[a:b])


def test_reference_randperm_contract(ref_C):
    for threads in (1, 4):
        out = ref_C.randperm(5000, threads, 7).numpy()
        assert operm.is_permutation(out)

"""GPU parity of the stand-alone kernels, called through the C ABI: gather and
permutations bit-exact, RowAdagrad / GEMM within 1e-5 relative of the oracle."""
import numpy as np
import pytest
import torch

from oracle import perm as operm
from oracle import step as ostep

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dim,n_rows,n", [(100, 1000, 4000), (3, 7, 20), (1024, 300, 513), (400, 64, 1), (6, 5, 0), (4096, 40, 100), (2050, 30, 64)])
def test_gather_bit_exact(pbg, dim, n_rows, n):
    say("gather", dim, n_rows, n)
    g = torch.Generator().manual_seed(dim)
    w = torch.randn(n_rows, dim, generator=g)
    idx = torch.randint(0, n_rows, (n,), generator=g)
    out = pbg.native.gather_rows(w.to(DEV), idx.to(DEV))
    assert torch.equal(out.cpu(), w[idx])
    # two-dimensional index (sample_entities' [C, U] layout)
    if n >= 4:
        idx2 = idx[: n // 2 * 2].view(2, -1)
        assert torch.equal(pbg.native.gather_rows(w.to(DEV), idx2.to(DEV)).cpu(), w[idx2])


def test_gather_out_of_range(pbg):
    w = torch.randn(5, 4, device=DEV)
    with pytest.raises(IndexError):
        pbg.native.gather_rows(w, torch.tensor([0, 5], device=DEV))


@pytest.mark.parametrize("m,n,k,batch,akm,bkm", [
    (50, 100, 100, 7, 0, 0), (100, 100, 50, 5, 1, 1), (50, 100, 100, 5, 0, 1),
    (130, 200, 33, 3, 0, 0), (1, 1, 1, 1, 0, 0), (200, 131, 257, 2, 1, 1), (17, 300, 64, 2, 0, 1),
    (256, 256, 300, 2, 1, 1), (64, 64, 16, 1, 0, 0),
    # aligned operands: the tiles that go from global memory straight into LDS, with
    # partial tiles along m, n and k in each of the four operand layouts
    (1000, 1100, 1024, 2, 0, 0), (1100, 1024, 1000, 2, 1, 1), (1000, 1024, 1100, 2, 0, 1), (132, 200, 36, 3, 1, 0),
    (128, 128, 16, 1, 0, 0), (200, 132, 20, 2, 0, 1), (97, 101, 64, 2, 0, 0), (130, 129, 16, 66000, 0, 0),
])
def test_gemm_against_float64(pbg, m, n, k, batch, akm, bkm):
    say("gemm", m, n, k, batch, akm, bkm)
    g = torch.Generator().manual_seed(m * 1000 + n)
    a = torch.randn((batch, k, m) if akm else (batch, m, k), generator=g)
    b = torch.randn((batch, k, n) if bkm else (batch, n, k), generator=g)
    c0 = torch.randn(batch, m, n, generator=g)
    am = a.transpose(1, 2) if akm else a
    bm = b if bkm else b.transpose(1, 2)
    for alpha, beta in ((1.0, 0.0), (0.5, 1.0)):
        want = alpha * torch.bmm(am.double(), bm.double()) + beta * c0.double()
        c = c0.clone().to(DEV)
        pbg.native.gemm(a.to(DEV), b.to(DEV), c, batch, m, n, k, m if akm else k, n if bkm else k, n,
                        a[0].numel(), b[0].numel(), m * n, akm, bkm, alpha, beta)
        got = c.cpu().double()
        scale = want.abs().max().item() + 1e-30
        assert (got - want).abs().max().item() <= 2e-6 * scale * max(1, k ** 0.5), (alpha, beta)


def test_bmm_nt_unaligned_dim(pbg):
    a = torch.randn(3, 5, 7)
    b = torch.randn(3, 6, 7)
    got = pbg.native.bmm_nt(a.to(DEV), b.to(DEV)).cpu()
    assert torch.allclose(got, torch.bmm(a, b.transpose(1, 2)), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dim,n_rows,n", [(100, 500, 4000), (1, 9, 30), (4, 50, 1), (1024, 40, 300), (10, 100000, 5000),
                                          (400, 3, 700), (4096, 30, 200), (2048, 5, 300), (2050, 20, 100), (1030, 9, 64)])
def test_row_adagrad_sparse(pbg, dim, n_rows, n):
    say("row_adagrad_sparse", dim, n_rows, n)
    g = torch.Generator().manual_seed(n)
    w = torch.randn(n_rows, dim, generator=g)
    gs = torch.rand(n_rows, generator=g)
    idx = torch.randint(0, n_rows, (n,), generator=g)
    vals = torch.randn(n, dim, generator=g)
    wd, gd = w.clone().to(DEV), gs.clone().to(DEV)
    pbg.native.row_adagrad_sparse(wd, gd, idx.to(DEV), vals.to(DEV), 0.1)
    ostep.row_adagrad_sparse(w, gs, torch.sparse_coo_tensor(idx.unsqueeze(0), vals, (n_rows, dim)), 0.1)
    assert torch.allclose(wd.cpu(), w, rtol=1e-5, atol=1e-6)
    assert torch.allclose(gd.cpu(), gs, rtol=1e-5, atol=1e-7)
    # a second step on top of the first (state carries over)
    pbg.native.row_adagrad_sparse(wd, gd, idx.to(DEV), vals.to(DEV), 0.1)
    ostep.row_adagrad_sparse(w, gs, torch.sparse_coo_tensor(idx.unsqueeze(0), vals, (n_rows, dim)), 0.1)
    assert torch.allclose(wd.cpu(), w, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("n, n_rows", [(1, 5), (15, 4), (16, 1000), (17, 3), (4000, 100000), (4001, 700), (8191, 50),
                                       (8192, 1 << 20), (8192, 9), (8193, 1000)])
def test_small_inputs_sort_in_one_launch_like_the_radix_sort(pbg, n, n_rows, monkeypatch):
    """Up to 8192 indices are sorted by one rank-counting launch; the result (order of equal indices
    included: the duplicates' sums are formed in that order) is that of the radix kernels bit for bit -- few
    rows so that runs are long, many so that there is none, sizes on both sides of the workgroup's 16 pairs
    and of the limit, and indices outside the table (parked behind it, ignored)."""
    say("rank sort", n, n_rows)
    g = torch.Generator().manual_seed(n + n_rows)
    w = torch.randn(n_rows, 12, generator=g)
    gs = torch.rand(n_rows, generator=g)
    idx = torch.randint(0, n_rows, (n,), generator=g)
    if n > 100:
        idx[::97] = n_rows + 5  # out of range
        idx[5::89] = -3
    vals = torch.randn(n, 12, generator=g)
    got = []
    for off in ("", "1"):
        if off:
            monkeypatch.setenv("PBG_DISABLE_RANK_SORT", off)
        wd, gd = w.clone().to(DEV), gs.clone().to(DEV)
        pbg.native.row_adagrad_sparse(wd, gd, idx.to(DEV), vals.to(DEV), 0.1)
        got.append((wd.cpu(), gd.cpu()))
    assert torch.equal(got[0][0], got[1][0]) and torch.equal(got[0][1], got[1][1])
    keep = (idx >= 0) & (idx < n_rows)
    ostep.row_adagrad_sparse(w, gs, torch.sparse_coo_tensor(idx[keep].unsqueeze(0), vals[keep], (n_rows, 12)), 0.1)
    assert torch.allclose(got[0][0], w, rtol=1e-5, atol=1e-6) and torch.allclose(got[0][1], gs, rtol=1e-5, atol=1e-7)


def test_row_adagrad_empty_and_dense(pbg):
    w = torch.randn(6, 5)
    gs = torch.rand(6)
    wd, gd = w.clone().to(DEV), gs.clone().to(DEV)
    pbg.native.row_adagrad_sparse(wd, gd, torch.empty(0, dtype=torch.int64, device=DEV),
                                  torch.empty(0, 5, device=DEV), 0.1)
    assert torch.equal(wd.cpu(), w)
    grad = torch.randn(6, 5)
    pbg.native.row_adagrad_dense(wd, gd, grad.to(DEV), 0.05)
    ostep.row_adagrad_dense(w, gs, grad, 0.05)
    assert torch.allclose(wd.cpu(), w, rtol=1e-6, atol=1e-7) and torch.allclose(gd.cpu(), gs, rtol=1e-6)
    p, s, gr = torch.randn(37), torch.rand(37), torch.randn(37)
    pd, sd = p.clone().to(DEV), s.clone().to(DEV)
    pbg.native.async_adagrad_dense(pd, sd, gr.to(DEV), 0.01)
    ostep.async_adagrad_dense(p, s, gr, 0.01)
    assert torch.allclose(pd.cpu(), p, rtol=1e-6, atol=1e-7) and torch.allclose(sd.cpu(), s, rtol=1e-6)


@pytest.mark.parametrize("n", [1, 2, 1000, 70001])
def test_permutation_helpers_bit_exact(pbg, n):
    say("perm", n)
    p = np.random.default_rng(n).permutation(n).astype(np.int64)
    tp = torch.from_numpy(p).to(DEV)
    assert np.array_equal(pbg.native.reverse_permutation(tp).cpu().numpy(), operm.reverse_permutation(p))
    # row widths on either side of every kernel's border: 4 / 8 bytes, up to 128 / 256 / 512 / 1024 bytes in
    # 16-byte words, wider than that, and widths that are no multiple of 16
    for shape, dtype in (((n, 100), torch.float32), ((n,), torch.float32), ((n,), torch.int64), ((n, 3), torch.float32),
                         ((n, 2, 2), torch.float64), ((n, 32), torch.float32), ((n, 36), torch.float32),
                         ((n, 64), torch.float32), ((n, 128), torch.float32), ((n, 132), torch.float32),
                         ((n, 256), torch.float32), ((n, 260), torch.float32), ((n, 1030), torch.float32)):
        if n * int(np.prod(shape[1:])) > 40_000_000:
            continue
        t = (torch.randn(shape) * 1000).to(dtype)
        want = operm.shuffle(t.numpy(), p)
        td = t.to(DEV)
        out = pbg.native.shuffle_rows_out(td, tp)   # into a second buffer, the input untouched
        assert np.array_equal(out.cpu().numpy(), want), (shape, dtype, "out of place")
        assert torch.equal(td.cpu(), t)
        pbg.native.shuffle_rows(td, tp)
        assert np.array_equal(td.cpu().numpy(), want), (shape, dtype)
    # undo with the reverse permutation (train_gpu.py:627-632)
    t = torch.randn(n, 8)
    td = t.to(DEV)
    pbg.native.shuffle_rows(td, tp)
    pbg.native.shuffle_rows(td, pbg.native.reverse_permutation(tp))
    assert torch.equal(td.cpu(), t)


def test_shuffle_rejects_bad_permutation(pbg):
    t = torch.randn(4, 4, device=DEV)
    with pytest.raises(ValueError):
        pbg.native.shuffle_rows(t, torch.tensor([0, 1, 2, 4], device=DEV))
    with pytest.raises(ValueError):
        pbg.native.shuffle_rows_out(t, torch.tensor([0, -1, 2, 3], device=DEV))
    both = torch.randn(8, 4, device=DEV)
    with pytest.raises(ValueError, match="overlap"):  # the out-of-place form needs two buffers
        pbg.native.shuffle_rows_out(both[:6], torch.arange(6, device=DEV), both[2:])


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 63, 64, 65, 5000, 65536, 65537, 200003, 1 << 20, 4_000_001])
def test_randperm_contract(pbg, n):
    """_C.randperm's contract (util.cpp:14-102; its bits depend on the thread count, so only the contract
    travels): a permutation, the same for the same seed, another for another seed, and uniform to first
    and second order -- where the first tenth of the elements lands, the differences of neighbouring
    outputs, and the joint position of neighbouring outputs on an 8 x 8 grid."""
    a = pbg.native.randperm(n, 7, DEV).cpu().numpy()
    assert operm.is_permutation(a)
    assert np.array_equal(a, pbg.native.randperm(n, 7, DEV).cpu().numpy())
    if n > 1000:
        b = pbg.native.randperm(n, 8, DEV).cpu().numpy()
        assert (a != b).mean() > 0.99

        def chi2(counts):
            expected = counts.sum() / counts.size
            return float(((counts - expected) ** 2 / expected).sum())

        for perm in (a, b):
            inv = np.empty(n, dtype=np.int64)
            inv[perm] = np.arange(n)
            assert chi2(np.bincount(inv[: n // 10] * 10 // n, minlength=10)) < 40                   # 9 dof
            assert chi2(np.bincount(np.diff(perm) % 16, minlength=16)) < 55                          # 15 dof
            assert chi2(np.bincount((perm[:-1] * 8 // n) * 8 + perm[1:] * 8 // n, minlength=64)) < 130  # 63 dof
            assert int((perm == np.arange(n)).sum()) < 12  # fixed points: Poisson(1)


def test_randperm_small_sizes_reach_every_permutation(pbg):
    """n = 4 has 24 permutations; over 600 seeds each must appear (expected 25 times)."""
    seen = {}
    for seed in range(600):
        key = tuple(pbg.native.randperm(4, seed, DEV).tolist())
        seen[key] = seen.get(key, 0) + 1
    assert len(seen) == 24 and min(seen.values()) >= 5, seen


@pytest.mark.parametrize("dynamic", [False, True])
@pytest.mark.parametrize("parts", [(1, 1), (2, 3), (8, 8)])
def test_sub_bucket_bit_exact(pbg, dynamic, parts):
    say("sub_bucket", dynamic, parts)
    rng = np.random.default_rng(5)
    n, n_rel = 20000, 3
    cl = [int(c) for c in rng.integers(50, 400, n_rel)]
    cr = [int(c) for c in rng.integers(50, 400, n_rel)]
    rel = rng.integers(0, n_rel, n).astype(np.int64)
    look = np.zeros(n, dtype=np.int64) if dynamic else rel
    lhs = (rng.random(n) * np.array(cl)[look]).astype(np.int64)
    rhs = (rng.random(n) * np.array(cr)[look]).astype(np.int64)
    pl = [rng.permutation(c).astype(np.int64) for c in cl]
    pr = [rng.permutation(c).astype(np.int64) for c in cr]
    lo, ro, relo, ranges = operm.sub_bucket(lhs, rhs, rel, cl, pl, cr, pr, parts[0], parts[1], dynamic)
    d = lambda x: torch.from_numpy(x).to(DEV)
    outs = [torch.empty(n, dtype=torch.int64, device=DEV) for _ in range(3)]
    offs = pbg.native.sub_bucket(
        d(lhs), d(rhs), d(rel), [d(x) for x in pl], [d(x) for x in pr],
        [-(-c // parts[0]) for c in cl], [-(-c // parts[1]) for c in cr], parts[0], parts[1], dynamic, *outs)
    assert np.array_equal(outs[0].cpu().numpy(), lo)
    assert np.array_equal(outs[1].cpu().numpy(), ro)
    assert np.array_equal(outs[2].cpu().numpy(), relo)
    offs = offs.cpu().numpy()
    for (i, j), (a, b) in ranges.items():
        assert (offs[i * parts[1] + j], offs[i * parts[1] + j + 1]) == (a, b)

"""Host-side mirror of the reference interface (no GPU needed): registries,
shape checks, containers, batching, argument validation.  The expectations are
the ones the reference's own unit tests state (test/test_util.py,
test/test_edgelist.py, test/test_entitylist.py, test/test_batching.py,
test/test_stats.py) or its documented error behaviour."""
import pytest
import torch


def test_plugin_registry(pbg):
    reg = pbg.plugin.PluginRegistry()

    @reg.register_as("a")
    class A:
        pass

    assert reg.get_class("a") is A
    reg.register("a", A)  # same class again is fine
    with pytest.raises(RuntimeError):
        reg.register("a", int)
    with pytest.raises(NotImplementedError, match="known names: a"):
        reg.get_class("b")
    assert sorted(pbg.operators.OPERATORS.registry) == ["affine", "complex_diagonal", "diagonal", "linear", "none", "translation"]
    assert sorted(pbg.operators.DYNAMIC_OPERATORS.registry) == sorted(pbg.operators.OPERATORS.registry)
    assert sorted(pbg.model.COMPARATORS.registry) == ["cos", "dot", "l2", "squared_l2"]
    assert sorted(pbg.losses.LOSS_FUNCTIONS.registry) == ["logistic", "ranking", "softmax"]
    with pytest.raises(TypeError):
        pbg.losses.LOSS_FUNCTIONS.get_class("ranking")()  # margin is keyword-required
    assert pbg.losses.LOSS_FUNCTIONS.get_class("softmax")(margin=0.1).loss_name == "softmax"


def test_split_almost_equally_and_rounding(pbg):
    sae = pbg.util.split_almost_equally
    assert list(sae(24, num_parts=4)) == [slice(0, 6), slice(6, 12), slice(12, 18), slice(18, 24)]
    assert list(sae(25, num_parts=4)) == [slice(0, 7), slice(7, 14), slice(14, 21), slice(21, 25)]
    assert list(sae(23, num_parts=4)) == [slice(0, 6), slice(6, 12), slice(12, 18), slice(18, 23)]
    assert list(sae(5, num_parts=4)) == [slice(0, 2), slice(2, 4), slice(4, 5), slice(5, 5)]
    assert list(sae(6, num_parts=5)) == [slice(0, 2), slice(2, 4), slice(4, 6), slice(6, 6), slice(6, 6)]
    r = pbg.util.round_up_to_nearest_multiple
    assert (r(24, 4), r(25, 4), r(23, 4)) == (24, 28, 24)


def test_match_shape(pbg):
    ms = pbg.util.match_shape
    t = torch.zeros(())
    assert ms(t) is None and ms(t, ...) is None
    for bad in (0, 1, -1):
        with pytest.raises(TypeError):
            ms(t, bad)
    t = torch.empty(2, 3, 4)
    assert ms(t, 2, 3, 4) is None
    assert ms(t, 2, -1, 4) == 3
    assert ms(t, -1, 3, -1) == (2, 4)
    assert ms(t, ..., 3, -1) == 4
    assert ms(t, 2, ...) is None
    assert ms(t, ..., 2, 3, 4) is None
    assert ms(t, -1, ..., -1) == (2, 4)
    with pytest.raises(TypeError):
        ms(t, 2, 3)
    with pytest.raises(TypeError):
        ms(t, 2, 3, 5)
    with pytest.raises(TypeError):
        ms(t, ..., 1, 2, 3, 4)
    with pytest.raises(RuntimeError):
        ms(t, ..., 3, ...)
    with pytest.raises(RuntimeError):
        ms(t, 2, 3.0, 4)


def test_entity_list(pbg):
    EL = pbg.entitylist.EntityList
    el = EL.from_tensor(torch.tensor([3, 4, 1, 0], dtype=torch.long))
    assert len(el) == 4 and len(EL.empty()) == 0
    assert el[1] == EL.from_tensor(torch.tensor([4]))
    assert el[1:3] == EL.from_tensor(torch.tensor([4, 1]))
    assert el[torch.tensor([2, 0])] == EL.from_tensor(torch.tensor([1, 3]))
    assert EL.cat([el[:2], el[2:]]) == el
    with pytest.raises(ValueError):
        el[::2]
    with pytest.raises(TypeError):
        EL(torch.tensor([1.0]))
    with pytest.raises(ValueError):
        EL.from_tensor(torch.zeros((2, 2), dtype=torch.long))
    with pytest.raises(NotImplementedError):
        el.to_tensor_list()


def test_edge_list(pbg):
    EL, ED = pbg.entitylist.EntityList, pbg.edgelist.EdgeList
    lhs = EL.from_tensor(torch.tensor([3, 4, 1, 0]))
    rhs = EL.from_tensor(torch.tensor([0, 2, 1, 3]))
    e = ED(lhs, rhs, torch.tensor([2, 0, 2, 1]))
    assert len(e) == 4 and not e.has_scalar_relation_type() and not e.has_weight()
    assert e[1:3] == ED(lhs[1:3], rhs[1:3], torch.tensor([0, 2]))
    assert e[torch.tensor([3, 0])] == ED(lhs[torch.tensor([3, 0])], rhs[torch.tensor([3, 0])], torch.tensor([1, 2]))
    with pytest.raises(RuntimeError):
        e.get_relation_type_as_scalar()
    s = ED(lhs, rhs, torch.tensor(3))
    assert s.has_scalar_relation_type() and s.get_relation_type_as_scalar() == 3 and s.get_relation_type() == 3
    assert s.get_relation_type_as_vector().tolist() == [3, 3, 3, 3]
    assert s[2:] .get_relation_type_as_scalar() == 3
    assert ED.cat([s[:2], s[2:]]).has_scalar_relation_type()
    assert not ED.cat([s[:2], ED(lhs[2:], rhs[2:], torch.tensor(1))]).has_scalar_relation_type()
    w = ED(lhs, rhs, torch.tensor(0), torch.tensor([1.0, 2.0, 3.0, 4.0]))
    assert w.has_weight() and w[1:3].weight.tolist() == [2.0, 3.0]
    assert ED(lhs, rhs, torch.tensor(0), torch.empty(0)).weight is None
    with pytest.raises(RuntimeError):
        ED.cat([w, s])
    with pytest.raises(ValueError):
        ED(lhs, rhs[:2], torch.tensor(0))
    with pytest.raises(ValueError):
        ED(lhs, rhs, torch.tensor([0, 1]))
    with pytest.raises(ValueError):
        ED(lhs, rhs, torch.zeros((4, 1), dtype=torch.long))
    with pytest.raises(TypeError):
        ED(lhs, rhs, torch.tensor(0.5))
    with pytest.raises(TypeError):
        ED(lhs.tensor, rhs, torch.tensor(0))
    with pytest.raises(TypeError):
        e[1.5]


def test_stats(pbg):
    S = pbg.stats.Stats
    a, b = S(count=2, loss=4.0, violators=2), S(count=6, loss=2.0, violators=4)
    assert S.sum([a, b]) == S(count=8, loss=6.0, violators=6)
    assert S.sum([a, b]).average() == S(count=8, loss=0.75, violators=0.75)
    assert S.average_list([a, b]) == S(count=8, loss=(4.0 * 2 + 2.0 * 6) / 8, violators=(2 * 2 + 4 * 6) / 8)
    assert S.from_dict(a.to_dict()) == a
    assert str(a) == "loss:  4 , violators:  2 , count:  2"
    with pytest.raises(ValueError):
        S.from_dict({"count": 1})


def test_group_by_relation_type_and_batchers(pbg):
    EL, ED = pbg.entitylist.EntityList, pbg.edgelist.EdgeList
    B = pbg.batching
    lhs = torch.tensor([93, 24, 13, 31, 70, 66, 77, 38, 5, 5])
    rhs = torch.tensor([90, 75, 9, 25, 23, 31, 49, 64, 42, 50])
    rel = torch.tensor([1, 0, 0, 1, 2, 2, 0, 0, 2, 2])
    edges = ED(EL.from_tensor(lhs), EL.from_tensor(rhs), rel)
    groups = B.group_by_relation_type(edges)
    assert groups == [
        ED(EL.from_tensor(torch.tensor([24, 13, 77, 38])), EL.from_tensor(torch.tensor([75, 9, 49, 64])), torch.tensor(0)),
        ED(EL.from_tensor(torch.tensor([93, 31])), EL.from_tensor(torch.tensor([90, 25])), torch.tensor(1)),
        ED(EL.from_tensor(torch.tensor([70, 66, 5, 5])), EL.from_tensor(torch.tensor([23, 31, 42, 50])), torch.tensor(2)),
    ]
    assert all(g.has_scalar_relation_type() for g in groups)
    assert B.group_by_relation_type(ED.empty()) == []
    const = ED(EL.from_tensor(lhs[:4]), EL.from_tensor(rhs[:4]), torch.tensor([3, 3, 3, 3]))
    assert B.group_by_relation_type(const) == [ED(const.lhs, const.rhs, torch.tensor(3))]
    mixed = list(B.batch_edges_mix_relation_types(edges, batch_size=4))
    assert [len(m) for m in mixed] == [4, 4, 2]
    assert mixed[0] == ED(EL.from_tensor(lhs[:4]), EL.from_tensor(rhs[:4]), rel[:4])
    torch.manual_seed(0)
    grouped = list(B.batch_edges_group_by_relation_type(edges, batch_size=3))
    assert sorted(len(g) for g in grouped) == [1, 1, 2, 3, 3]
    assert all(g.has_scalar_relation_type() for g in grouped)
    seen = sorted((int(l), int(r), g.get_relation_type_as_scalar()) for g in grouped
                  for l, r in zip(g.lhs.tensor, g.rhs.tensor))
    assert seen == sorted(zip(lhs.tolist(), rhs.tolist(), rel.tolist()))


def test_relation_batches_of_a_group_beyond_2_pow_24_edges(pbg, monkeypatch):
    """A relation type with more than 2**24 edges (a single-relation bucket of the
    LiveJournal example has 62 M): a float32 count of the edges left cannot step by
    one there.  Groups are stand-ins that only know their length."""
    import itertools
    B = pbg.batching

    class Span:
        def __init__(self, n):
            self.n = n

        def __len__(self):
            return self.n

        def __getitem__(self, sl):
            start, stop, _ = sl.indices(self.n)
            return Span(max(stop - start, 0))

    sizes = [2 ** 24 + 3, 5, 2 ** 24 + 1]
    monkeypatch.setattr(B, "group_by_relation_type", lambda edges: [Span(n) for n in sizes])
    torch.manual_seed(0)
    batch_size = 4099
    want = sum(-(-n // batch_size) for n in sizes)
    got = list(itertools.islice(B.batch_edges_group_by_relation_type(None, batch_size=batch_size), want + 10))
    assert len(got) == want
    assert sum(len(g) for g in got) == sum(sizes)
    assert all(0 < len(g) <= batch_size for g in got)


def test_argument_validation_without_gpu(pbg):
    with pytest.raises(ValueError, match="even dimension"):
        pbg.operators.ComplexDiagonalOperator(3)
    with pytest.raises(ValueError, match="even dimension"):
        pbg.operators.ComplexDiagonalDynamicOperator(5, 2)
    with pytest.raises(NotImplementedError):
        pbg.operators.instantiate_operator("rotation", pbg.types.Side.RHS, 0, 4)
    aff = pbg.operators.instantiate_operator("affine", pbg.types.Side.RHS, 0, 4)
    assert torch.equal(aff.linear_transformation, torch.eye(4)) and torch.equal(aff.translation, torch.zeros(4))
    aff = pbg.operators.instantiate_operator("affine", pbg.types.Side.LHS, 3, 4)
    assert tuple(aff.linear_transformations.shape) == (3, 4, 4) and tuple(aff.translations.shape) == (3, 4)
    assert pbg.operators.instantiate_operator("linear", pbg.types.Side.LHS, 0, 4) is None
    op = pbg.operators.instantiate_operator("linear", pbg.types.Side.LHS, 7, 4)
    assert tuple(op.linear_transformations.shape) == (7, 4, 4)
    assert torch.equal(op.linear_transformations[3], torch.eye(4))
    assert torch.equal(pbg.operators.DiagonalOperator(3).diagonal, torch.ones(3))
    assert torch.equal(pbg.operators.TranslationDynamicOperator(3, 2).translations, torch.zeros(2, 3))
    with pytest.raises(ValueError, match="2D"):
        pbg.row_adagrad.RowAdagrad([torch.nn.Parameter(torch.zeros(3))])
    opt = pbg.row_adagrad.RowAdagrad([torch.nn.Parameter(torch.zeros(5, 3))], lr=0.1)
    (p,) = opt.param_groups[0]["params"]
    assert tuple(opt.state[p]["sum"].shape) == (5,)
    assert "sum" in str(opt.state_dict()["state"][0].keys())
    # shuffle argument checks (util.cpp:131-161) fire before anything touches the GPU
    C = pbg._C
    with pytest.raises(ValueError, match="int64"):
        C.shuffle(torch.zeros(3, 2), torch.zeros(3), 1)
    with pytest.raises(ValueError, match="one dimension"):
        C.shuffle(torch.zeros(3, 2), torch.zeros((3, 1), dtype=torch.long), 1)
    with pytest.raises(ValueError, match="same number"):
        C.shuffle(torch.zeros(3, 2), torch.zeros(2, dtype=torch.long), 1)
    with pytest.raises(ValueError, match="contiguous"):
        C.shuffle(torch.zeros(3, 2, 4).transpose(1, 2), torch.zeros(3, dtype=torch.long), 1)
    C.shuffle(torch.zeros(0, 2), torch.zeros(0, dtype=torch.long), 1)  # empty: no-op
    with pytest.raises(RuntimeError, match="Inconsistent"):
        C.sub_bucket(None, None, None, [1], [torch.zeros(1)], [1, 2], [torch.zeros(1)], None, None, None, 1, 1, 1, False)


def test_no_cpu_fallback(pbg):
    """The product has no CPU path: CPU tensors are refused, loudly."""
    with pytest.raises(TypeError, match="GPU"):
        pbg.native.gather_rows(torch.zeros(3, 4), torch.zeros(2, dtype=torch.long))
    with pytest.raises(TypeError, match="GPU"):
        pbg.operators.DiagonalOperator(3)(torch.zeros(2, 3))
    with pytest.raises(TypeError, match="GPU"):
        pbg.losses.SoftmaxLossFunction()(torch.zeros(2), torch.zeros(2, 3), None)
    with pytest.raises(TypeError, match="GPU"):
        pbg.model.DotComparator()(torch.zeros(1, 2, 3), torch.zeros(1, 2, 3), torch.zeros(1, 4, 3), torch.zeros(1, 4, 3))


def test_model_argument_errors(pbg):
    M, C = pbg.model, pbg.config
    rel = [C.RelationSchema(name="r", lhs="e", rhs="e", operator="translation")]
    ent = {"e": C.EntitySchema()}
    mk = lambda **kw: M.MultiRelationEmbedder(4, rel, ent, 2, 2, False, False, [None],
                                              [pbg.operators.TranslationOperator(4)], M.DotComparator(), **kw)
    with pytest.raises(NotImplementedError):
        mk(regularizer=object())
    # model.py:444: kept, and handed on to every step the model describes
    assert mk(half_precision=True).step_spec(0, 3, 4).half_precision and not mk().step_spec(0, 3, 4).half_precision
    capped = mk(max_norm=1.0)  # model.py:443-451: handed on to every embedding module
    capped.set_embeddings("e", pbg.types.Side.LHS, torch.nn.Parameter(torch.zeros(5, 4)))
    assert capped.lhs_embs["emb_e"].max_norm == 1.0 and capped.step_spec(0, 3, 4).max_norm == 1.0
    with_global = mk(global_emb=True)  # model.py:433-439: a zero vector per entity type
    assert list(with_global.global_embs) == ["emb_e"] and float(with_global.global_embs["emb_e"].abs().sum()) == 0.0
    assert mk().global_embs is None
    model = mk()
    EL, ED = pbg.entitylist.EntityList, pbg.edgelist.EdgeList
    w = torch.nn.Parameter(torch.zeros(5, 4))
    model.set_embeddings("e", pbg.types.Side.LHS, w)
    model.set_embeddings("e", pbg.types.Side.RHS, w)
    edges = ED(EL.from_tensor(torch.tensor([0, 1])), EL.from_tensor(torch.tensor([2, 3])), torch.tensor([0, 0]))
    with pytest.raises(TypeError, match="same relation"):
        model(edges)
    dyn = M.MultiRelationEmbedder(4, rel, ent, 2, 2, False, False, [pbg.operators.TranslationDynamicOperator(4, 3)],
                                  [pbg.operators.TranslationDynamicOperator(4, 3)], M.DotComparator(), num_dynamic_rels=3)
    dyn.set_embeddings("e", pbg.types.Side.LHS, w)
    dyn.set_embeddings("e", pbg.types.Side.RHS, w)
    with pytest.raises(TypeError, match="relation for each"):
        dyn(ED(edges.lhs, edges.rhs, torch.tensor(0)))
    bad = M.MultiRelationEmbedder(4, rel, ent, 2, 2, False, False, [pbg.operators.TranslationOperator(4)],
                                  [pbg.operators.TranslationOperator(4)], M.DotComparator())
    bad.set_embeddings("e", pbg.types.Side.LHS, w)
    bad.set_embeddings("e", pbg.types.Side.RHS, w)
    with pytest.raises(RuntimeError, match="right-hand side operator"):
        bad(ED(edges.lhs, edges.rhs, torch.tensor(0)))


def test_bench_refuses_more_than_one_gpu():
    import pathlib
    import subprocess
    import sys

    root = pathlib.Path(__file__).resolve().parent.parent
    out = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 2
    assert "ONE GPU" in out.stderr

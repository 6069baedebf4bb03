"""The oracle against every literal vector the reference's own tests hold for
the path (test/test_model.py, test/test_losses.py), at the reference's own
tolerance (rtol = atol = 5e-5)."""
import pytest
import torch

from oracle import step


def close(a, b, tol):
    return torch.allclose(a, torch.as_tensor(b, dtype=torch.float32), rtol=tol, atol=tol, equal_nan=True)


def test_operators(golden):
    tol = golden["tolerance"]
    for case in golden["operators"]:
        x = torch.tensor(case["input"], requires_grad=True)
        params = {}
        for k, v in case["params"].items():
            t = torch.tensor(v)
            if case["dynamic"]:
                # the reference's dynamic parameter names are plural
                k = {"diagonals": "diagonal", "translations": "translation",
                     "linear_transformations": "linear_transformation"}.get(k, k)
            else:
                t = t.unsqueeze(0)
            params[k] = t.requires_grad_(True)
        rel = torch.tensor(case["rel"]) if case["dynamic"] else 0
        y = step.apply_operator(case["name"], x, params, rel)
        assert y.shape == x.shape
        assert close(y, case["expected"], tol), (case["name"], case["dynamic"])
        y.sum().backward()
        assert (x.grad != 0).any()
        for p in params.values():
            assert (p.grad != 0).any()


def test_comparators(golden):
    tol = golden["tolerance"]
    for case in golden["comparators"]:
        ts = [torch.tensor(case[k], requires_grad=True) for k in ("lhs_pos", "rhs_pos", "lhs_neg", "rhs_neg")]
        prep = [step.comparator_prepare(case["name"], t) for t in ts]
        pos, lneg, rneg = step.comparator_scores(case["name"], *prep)
        assert close(pos, case["pos"], tol), case["ref"]
        assert close(lneg, case["lhs_neg_scores"], tol), case["ref"]
        assert close(rneg, case["rhs_neg_scores"], tol), case["ref"]
        (pos.sum() + lneg.sum() + rneg.sum()).backward()
        for t in ts:
            assert (t.grad != 0).any()


def test_losses(golden):
    tol = golden["tolerance"]
    for case in golden["losses"]:
        pos = torch.tensor(case["pos"], dtype=torch.float32, requires_grad=True)
        if "neg_shape" in case:
            neg = torch.empty(case["neg_shape"], requires_grad=True)
        else:
            neg = torch.tensor(case["neg"], dtype=torch.float32).view(len(case["pos"]), -1).requires_grad_(True)
        w = torch.tensor(case["weight"]) if case["weight"] is not None else None
        loss = step.loss_value(case["name"], pos, neg, w, margin=case["margin"] or 0.1)
        assert loss.dim() == 0
        assert close(loss, case["expected"], tol), (case["name"], case["case"], float(loss))
        loss.backward()


def test_biased_comparators(golden):
    """BiasedComparator (model.py:306-344) against the reference's own vectors."""
    tol = golden["tolerance"]
    for case in golden["biased_comparators"]:
        ts = [torch.tensor(case[k], requires_grad=True) for k in ("lhs_pos", "rhs_pos", "lhs_neg", "rhs_neg")]
        prep = [step.biased_prepare(case["name"], t) for t in ts]
        pos, lneg, rneg = step.biased_scores(case["name"], *prep)
        assert close(pos, case["pos"], tol), case["ref"]
        assert close(lneg, case["lhs_neg_scores"], tol), case["ref"]
        assert close(rneg, case["rhs_neg_scores"], tol), case["ref"]
        (pos.sum() + lneg.sum() + rneg.sum()).backward()
        for t in ts:
            assert (t.grad != 0).any()


def test_gather(golden):
    g = golden["gather"]
    w = torch.tensor(g["table"], requires_grad=True)
    out = torch.nn.functional.embedding(torch.tensor(g["index"]), w, sparse=True)
    assert torch.equal(out, torch.tensor(g["expected"]))
    # sample_entities draws torch.randint(0, E, (C, U)) on the global generator
    torch.manual_seed(g["sample_seed"])
    idx = torch.randint(low=0, high=w.shape[0], size=tuple(g["sample_shape"]))
    assert torch.equal(w.detach()[idx], torch.tensor(g["sample_expected"]))


def test_gather_max_norm(golden):
    """The oracle's lookup with max_norm (F.embedding(max_norm=...) inside
    step.forward_backward) against the reference's vectors: the looked-up rows
    come back renormalised and the table keeps them."""
    g, m = golden["gather"], golden["gather"]["max_norm"]
    tol = golden["tolerance"]
    cfg = step.StepConfig(dim=3, num_batch_negs=3, num_uniform_negs=0, max_norm=m["max_norm"], lr=0.0)
    st = step.make_state(cfg, torch.tensor(g["table"]))
    idx = torch.tensor(m["index"])
    step.forward_backward(cfg, st, idx, idx, 0, None, None)
    assert close(st.w_lhs[idx], m["expected"], tol)
    assert close(st.w_lhs[1], g["table"][1], 0.0)  # not looked up: left alone
    st = step.make_state(cfg, torch.tensor(g["table"]))
    every = torch.arange(3)
    step.forward_backward(cfg, st, every, every, 0, None, None)
    assert close(st.w_lhs, m["all_entities_expected"], tol)


def test_operator_errors():
    with pytest.raises(ValueError):
        step.init_operator_params("complex_diagonal", 3, 1)
    with pytest.raises(NotImplementedError):
        step.init_operator_params("nope", 4, 1)

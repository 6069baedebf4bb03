"""The C-ABI library loads and exports every symbol include/pbg_hip.h declares
(no compute calls: this runs without a GPU)."""
import pathlib
import re

ROOT = pathlib.Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "pbg_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pbg_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(pbg):
    lib = pbg._lib.lib()
    names = declared_symbols()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), name
    assert set(names) == set(pbg._lib.SIGNATURES), set(names) ^ set(pbg._lib.SIGNATURES)
    assert lib.pbg_version() >= 1


def test_struct_sizes_match_the_header(pbg):
    import ctypes

    # 16 4-byte fields, two int64, five 4-byte fields and 4 bytes of padding: 16 * 4 + 16 + 5 * 4 + 4
    assert ctypes.sizeof(pbg._lib.StepDesc) == 104
    # 22 pointers + workspace_bytes, then sample_uniform (4 + 4 padding) and uniform_seed
    assert ctypes.sizeof(pbg._lib.StepBuffers) == 30 * 8
    lib = pbg._lib.lib()
    assert lib.pbg_sizeof_step_desc() == ctypes.sizeof(pbg._lib.StepDesc)
    assert lib.pbg_sizeof_step_buffers() == ctypes.sizeof(pbg._lib.StepBuffers)


def test_argument_errors_need_no_gpu(pbg):
    import ctypes

    lib = pbg._lib.lib()
    assert lib.pbg_gather_rows(None, 10, 4, None, 3, None, None, None) == pbg._lib.PBG_ERR_INVALID
    assert b"null" in lib.pbg_last_error()
    assert lib.pbg_gather_rows(None, 10, 4, None, 0, None, None, None) == pbg._lib.PBG_OK
    d = pbg._lib.StepDesc()
    d.dim, d.num_workers, d.batch_size = 5, 1, 10
    d.num_batch_negs, d.num_uniform_negs = 2, 2
    d.op = pbg._lib.OPERATOR_CODES["complex_diagonal"]
    d.num_relations, d.num_lhs_rows, d.num_rhs_rows = 1, 10, 10
    assert lib.pbg_train_step_workspace_bytes(ctypes.byref(d)) == 0
    assert b"even dimension" in lib.pbg_last_error()
    d.dim = 6
    assert lib.pbg_train_step_workspace_bytes(ctypes.byref(d)) > 0
    # rows of up to 4096 floats are taken; the next even width is refused with a message that says so
    d.dim = 4096
    assert lib.pbg_train_step_workspace_bytes(ctypes.byref(d)) > 0
    d.dim = 4098
    assert lib.pbg_train_step_workspace_bytes(ctypes.byref(d)) == 0
    assert b"[1, 4096]" in lib.pbg_last_error()
    assert lib.pbg_row_adagrad_sparse_workspace_bytes(1000) > 1000 * 24


def test_newer_step_fields_are_validated_without_a_gpu(pbg):
    import ctypes

    L = pbg._lib
    lib = L.lib()

    def desc(**kw):
        d = L.StepDesc()
        d.dim, d.num_workers, d.batch_size = 8, 1, 10
        d.num_batch_negs, d.num_uniform_negs = 2, 2
        d.num_relations, d.num_lhs_rows, d.num_rhs_rows = 1, 100, 100
        d.shared_table = 1
        for k, v in kw.items():
            setattr(d, k, v)
        return d

    size = lambda d: lib.pbg_train_step_workspace_bytes(ctypes.byref(d))
    plain = size(desc())
    assert plain > 0
    # bias: with every comparator (l2 keeps dLoss/dscore in a matrix of its own) and with a regularizer,
    # not with a single coordinate
    # (compared on the staged kernels, which a call with one relation per edge takes like a call with a bias)
    assert size(desc(bias=1, dynamic=1)) > size(desc(dynamic=1)) > 0
    assert size(desc(bias=1)) > 0
    assert size(desc(bias=1, comparator=L.COMPARATOR_CODES["l2"])) > size(desc(bias=1, comparator=L.COMPARATOR_CODES["squared_l2"]))
    assert size(desc(bias=1, regularization_coef=0.1, op=L.OPERATOR_CODES["diagonal"])) > 0
    assert size(desc(bias=1, dim=1)) == 0 and b"bias" in lib.pbg_last_error()
    # affine: two parameter slots, no regularizer (operators.py:40)
    assert size(desc(op=L.OPERATOR_CODES["affine"])) > size(desc(op=L.OPERATOR_CODES["linear"])) > 0
    assert size(desc(op=L.OPERATOR_CODES["affine"], regularization_coef=0.1)) == 0
    assert size(desc(op=6)) == 0 and b"unknown operator" in lib.pbg_last_error()
    # all_negs: needs no negatives' counts; the score matrices grow with the tables
    assert size(desc(all_negs=1, num_batch_negs=0, num_uniform_negs=0)) > size(desc(dynamic=1))
    assert size(desc(num_batch_negs=0, num_uniform_negs=0)) == 0
    assert size(desc(all_negs=1, num_lhs_rows=1 << 25, num_rhs_rows=1 << 25)) == 0
    # max_norm adds the per-slot scales
    assert size(desc(max_norm=1.0)) > plain
    # the renormalisation entry point
    assert lib.pbg_embedding_renorm_workspace_bytes(1000, 100) >= 1000 * 101 * 4
    assert lib.pbg_embedding_renorm(None, 10, 4, None, 0, 1.0, None, 0, None) == L.PBG_OK
    assert lib.pbg_embedding_renorm(None, 10, 4, None, 3, 1.0, None, 0, None) == L.PBG_ERR_INVALID
    assert lib.pbg_embedding_renorm(None, 10, 4, None, 3, 0.0, None, 0, None) == L.PBG_ERR_INVALID

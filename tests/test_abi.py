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

    # 15 x 4-byte fields + one 4-byte field, then two int64: 16 * 4 + 16
    assert ctypes.sizeof(pbg._lib.StepDesc) == 96
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
    assert lib.pbg_row_adagrad_sparse_workspace_bytes(1000) > 1000 * 24

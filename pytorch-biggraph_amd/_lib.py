"""ctypes binding of libpbg_hip.so (the C ABI declared in include/pbg_hip.h).

There is no CPU fallback: every call needs the built library and a GPU, and
`lib()` raises if the library is missing.
"""
import ctypes
import pathlib
from ctypes import POINTER, c_char_p, c_float, c_int32, c_int64, c_size_t, c_uint64, c_void_p

_HERE = pathlib.Path(__file__).resolve().parent
LIB_PATH = _HERE / "libpbg_hip.so"

OPERATOR_CODES = {"none": 0, "diagonal": 1, "translation": 2, "linear": 3, "complex_diagonal": 4, "affine": 5}
COMPARATOR_CODES = {"dot": 0, "cos": 1, "l2": 2, "squared_l2": 3}
LOSS_CODES = {"ranking": 0, "logistic": 1, "softmax": 2}

PBG_OK = 0
PBG_ERR_INVALID = -1
PBG_ERR_WORKSPACE = -2
PBG_ERR_LAUNCH = -3
PBG_ERR_UNSUPPORTED = -4


class StepDesc(ctypes.Structure):
    """pbg_step_desc"""

    _fields_ = [
        ("dim", c_int32),
        ("num_workers", c_int32),
        ("batch_size", c_int32),
        ("num_batch_negs", c_int32),
        ("num_uniform_negs", c_int32),
        ("disable_lhs_negs", c_int32),
        ("disable_rhs_negs", c_int32),
        ("op", c_int32),
        ("dynamic", c_int32),
        ("num_relations", c_int32),
        ("comparator", c_int32),
        ("loss", c_int32),
        ("margin", c_float),
        ("lr", c_float),
        ("relation_lr", c_float),
        ("shared_table", c_int32),
        ("num_lhs_rows", c_int64),
        ("num_rhs_rows", c_int64),
        ("regularization_coef", c_float),
        ("max_norm", c_float),
        ("bias", c_int32),
        ("all_negs", c_int32),
        ("half_precision", c_int32),
    ]


class StepBuffers(ctypes.Structure):
    """pbg_step_buffers"""

    _fields_ = [
        ("w_lhs", c_void_p), ("g_lhs", c_void_p), ("w_rhs", c_void_p), ("g_rhs", c_void_p),
        ("lhs", c_void_p), ("rhs", c_void_p), ("rel", c_void_p),
        ("uniform_lhs", c_void_p), ("uniform_rhs", c_void_p),
        ("edge_weight", c_void_p), ("relation_weights", c_void_p),
        ("rhs_op_p0", c_void_p), ("rhs_op_p1", c_void_p), ("rhs_op_s0", c_void_p), ("rhs_op_s1", c_void_p),
        ("lhs_op_p0", c_void_p), ("lhs_op_p1", c_void_p), ("lhs_op_s0", c_void_p), ("lhs_op_s1", c_void_p),
        ("loss_out", c_void_p), ("violators_out", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("sample_uniform", c_int32), ("uniform_seed", c_uint64), ("reg_out", c_void_p),
        ("lhs_global", c_void_p), ("rhs_global", c_void_p), ("lhs_global_sum", c_void_p), ("rhs_global_sum", c_void_p),
    ]


# name -> (restype, argtypes); every symbol include/pbg_hip.h declares
SIGNATURES = {
    "pbg_version": (c_int32, []),
    "pbg_last_error": (c_char_p, []),
    "pbg_gather_rows": (c_int32, [c_void_p, c_int64, c_int32, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "pbg_embedding_renorm_workspace_bytes": (c_size_t, [c_int64, c_int32]),
    "pbg_embedding_renorm": (c_int32, [c_void_p, c_int64, c_int32, c_void_p, c_int64, c_float, c_void_p, c_size_t, c_void_p]),
    "pbg_row_adagrad_sparse_workspace_bytes": (c_size_t, [c_int64]),
    "pbg_row_adagrad_sparse": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int64,
                                         c_float, c_void_p, c_size_t, c_void_p]),
    "pbg_row_adagrad_sparse_static_max_indices": (c_int64, []),
    "pbg_row_adagrad_sparse_static": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int64,
                                                c_float, c_void_p]),
    "pbg_row_adagrad_dense": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_float, c_void_p]),
    "pbg_async_adagrad_dense": (c_int32, [c_void_p, c_void_p, c_void_p, c_int64, c_float, c_float, c_void_p]),
    "pbg_gemm_f32": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
                               c_int32, c_int64, c_int64, c_int64, c_int32, c_int32, c_float, c_float, c_void_p]),
    "pbg_gemm_f16": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
                               c_int32, c_int64, c_int64, c_int64, c_int32, c_int32, c_float, c_float, c_void_p]),
    "pbg_sizeof_step_desc": (c_size_t, []),
    "pbg_sizeof_step_buffers": (c_size_t, []),
    "pbg_sample_uniform_negatives": (c_int32, [c_uint64, c_int32, c_int64, c_int64, c_void_p, c_void_p]),
    "pbg_train_step_workspace_bytes": (c_size_t, [POINTER(StepDesc)]),
    "pbg_train_step": (c_int32, [POINTER(StepDesc), POINTER(StepBuffers), c_void_p]),
    "pbg_train_step_num_stages": (c_int32, []),
    "pbg_train_step_is_fused": (c_int32, [POINTER(StepDesc)]),
    "pbg_train_step_route": (c_int32, [POINTER(StepDesc)]),
    "pbg_train_step_profile": (c_int32, [POINTER(StepDesc), POINTER(StepBuffers), c_void_p, POINTER(c_float)]),
    "pbg_model_ranks": (c_int32, [POINTER(StepDesc), POINTER(StepBuffers), c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_int64, c_uint64, c_void_p, c_void_p]),
    "pbg_model_forward": (c_int32, [POINTER(StepDesc), POINTER(StepBuffers), c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_void_p]),
    "pbg_operator_forward": (c_int32, [c_int32, c_int32, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                       c_void_p, c_void_p]),
    "pbg_operator_backward": (c_int32, [c_int32, c_int32, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "pbg_comparator_prepare": (c_int32, [c_int32, c_int32, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "pbg_comparator_prepare_backward": (c_int32, [c_int32, c_int32, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                                  c_void_p]),
    "pbg_comparator_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32]),
    "pbg_comparator_forward": (c_int32, [c_int32] * 6 + [c_void_p] * 8 + [c_size_t, c_void_p]),
    "pbg_comparator_backward": (c_int32, [c_int32] * 6 + [c_void_p] * 15 + [c_size_t, c_void_p]),
    "pbg_loss_forward": (c_int32, [c_int32, c_float, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p]),
    "pbg_loss_backward": (c_int32, [c_int32, c_float, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_void_p]),
    "pbg_reverse_permutation": (c_int32, [c_void_p, c_int64, c_void_p, c_void_p]),
    "pbg_shuffle_rows": (c_int32, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "pbg_shuffle_rows_out": (c_int32, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "pbg_randperm_workspace_bytes": (c_size_t, [c_int64]),
    "pbg_randperm": (c_int32, [c_int64, c_uint64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "pbg_sub_bucket_workspace_bytes": (c_size_t, [c_int64]),
    "pbg_sub_bucket": (c_int32, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_void_p, c_size_t, c_void_p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python {_HERE / 'csrc' / 'build.py'}` "
                "(there is no CPU fallback for this package)"
            )
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if handle.pbg_sizeof_step_desc() != ctypes.sizeof(StepDesc) or \
                handle.pbg_sizeof_step_buffers() != ctypes.sizeof(StepBuffers):
            raise RuntimeError(f"{LIB_PATH} was built from another include/pbg_hip.h than this binding: rebuild it")
        _lib = handle
    return _lib


class PbgError(RuntimeError):
    pass


def check(status: int) -> None:
    """Maps a pbg_status to the exception type the reference raises for the
    same mistake (ValueError / TypeError come from the Python layer; the C
    layer only reports invalid arguments, workspace and launch failures)."""
    if status == PBG_OK:
        return
    msg = lib().pbg_last_error().decode("utf-8", "replace")
    if status == PBG_ERR_INVALID:
        raise ValueError(msg)
    if status == PBG_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise PbgError(f"pbg status {status}: {msg}")

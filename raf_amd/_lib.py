"""ctypes bindings of the C ABI declared in include/rafhip_optim.h.

The libraries are built in-tree by ``python -m raf_amd.build`` (hipcc, gfx950).  Loading fails
loudly if they are missing: there is no CPU or eager fallback anywhere in this package.
"""
from __future__ import annotations

import ctypes
from ctypes import (POINTER, Structure, c_char_p, c_double, c_float, c_int, c_int32, c_int64,
                    c_void_p)
from pathlib import Path

LIB_DIR = Path(__file__).resolve().parent / "lib"
OPTIM_LIB = LIB_DIR / "libraf_hip_optim.so"
DIALECT_LIB = LIB_DIR / "libraf_hip_dialect.so"
GLUE_LIB = LIB_DIR / "_torch_glue.so"

RAFHIP_OK = 0
RAFHIP_ERR_INVALID_ARG = 1
RAFHIP_ERR_UNSUPPORTED = 2
RAFHIP_ERR_WORKSPACE = 3
RAFHIP_ERR_HIP = 4
RAFHIP_ERR_NO_DEVICE = 5
RAFHIP_ERR_HOST = 6

RAFHIP_F32 = 0
RAFHIP_F16 = 1
RAFHIP_BF16 = 2
RAFHIP_F64 = 3

RAFHIP_LANS_PHASED = 0
RAFHIP_LANS_PIPELINED = 1
RAFHIP_TABLE_SLOTS = 4  # device pointer tables per plan
RAFHIP_LANS_STATIC_SCRATCH_BYTES = 8 * 1024 * 1024


class RafHipError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"rafhip status {status}: {message}")
        self.status = status
        self.message = message


class LansHParams(Structure):
    """``rafhip_lans_hparams``: schema order of ``raf.op.lans``
    (scripts/src_codegen/def_schema.py:685-693 in the reference) plus ``grad_unscale``."""

    _fields_ = [
        ("learning_rate", c_float),
        ("beta1", c_float),
        ("beta2", c_float),
        ("eps", c_float),
        ("bias_correction", c_int32),
        ("weight_decay", c_float),
        ("grad_averaging", c_int32),
        ("mode", c_int32),
        ("normalize_grad", c_int32),
        ("grad_unscale", c_float),
    ]


class LansPlanOptions(Structure):
    """``rafhip_lans_plan_options``; ``defaults()`` gives the struct with every field at "the
    library's choice"."""

    _fields_ = [
        ("schedule", c_int32),
        ("round_slices", c_int32),
        ("group_elements", c_int64),
        ("stream_from_elements", c_int64),
        ("stream_hold_items", c_int32),
        ("blocks_per_cu", c_int32),
        ("resident_mib", c_int32),
        ("apply_slice_shift", c_int32),
        ("spin_limit", c_int64),
    ]

    @classmethod
    def defaults(cls, **fields):
        o = cls()
        optim().rafhip_lans_default_plan_options(ctypes.byref(o))
        for name, value in fields.items():
            if name not in dict(cls._fields_):
                raise TypeError(f"no plan option {name!r}")
            setattr(o, name, int(value))
        return o


# name -> (restype, argtypes); every symbol the header declares.
OPTIM_SYMBOLS = {
    "rafhip_abi_version": (c_int, []),
    "rafhip_last_error": (c_char_p, []),
    "rafhip_device_count": (c_int, []),
    "rafhip_sgd_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_double,
                               c_double, c_void_p]),
    "rafhip_sgd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_double,
                           c_double, c_void_p]),
    "rafhip_lans_default_hparams": (None, [POINTER(LansHParams)]),
    "rafhip_lans_chunk_elements": (c_int32, [c_int64]),
    "rafhip_lans_pass_a_unit_elements": (c_int32, [c_int64]),
    "rafhip_lans_pipeline_order": (c_int, [c_int32, POINTER(c_int64), c_int64, POINTER(c_int32), c_int64,
                                           POINTER(c_int64)]),
    "rafhip_lans_plan_set_schedule": (c_int, [c_void_p, c_int32]),
    "rafhip_lans_plan_schedule": (c_int32, [c_void_p]),
    "rafhip_lans_query_layout": (c_int, [c_int32, POINTER(c_int64), POINTER(c_int64),
                                         POINTER(c_int64)]),
    "rafhip_lans_plan_create": (c_int, [c_int32, POINTER(c_int64), c_int32, POINTER(c_void_p)]),
    "rafhip_lans_default_plan_options": (None, [POINTER(LansPlanOptions)]),
    "rafhip_lans_plan_create_with": (c_int, [c_int32, POINTER(c_int64), c_int32, POINTER(LansPlanOptions),
                                             POINTER(c_void_p)]),
    "rafhip_lans_pipeline_order_with": (c_int, [c_int32, POINTER(c_int64), POINTER(LansPlanOptions),
                                                POINTER(c_int32), c_int64, POINTER(c_int64)]),
    "rafhip_lans_plan_destroy": (c_int, [c_void_p]),
    "rafhip_lans_workspace_bytes": (c_int64, [c_void_p]),
    "rafhip_lans_plan_num_tensors": (c_int32, [c_void_p]),
    "rafhip_lans_plan_num_chunks": (c_int64, [c_void_p]),
    "rafhip_lans_plan_total_elements": (c_int64, [c_void_p]),
    "rafhip_lans_plan_table_uploads": (c_int64, [c_void_p]),
    "rafhip_lans_step": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                 POINTER(c_void_p), c_void_p, c_int32, POINTER(LansHParams),
                                 c_void_p, c_int64, c_void_p]),
    "rafhip_lans_step_mixed": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                       POINTER(c_void_p), POINTER(c_void_p), c_int32, c_void_p, c_int32,
                                       POINTER(LansHParams), c_void_p, c_int64, c_void_p]),
    "rafhip_lans_step_noalloc": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                         POINTER(c_void_p), POINTER(c_void_p), c_int32, c_void_p, c_int32,
                                         POINTER(LansHParams), c_void_p]),
    "rafhip_lans_plan_bind": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                      POINTER(c_void_p), POINTER(c_void_p), c_int32]),
    "rafhip_lans_step_bound": (c_int, [c_void_p, c_void_p, c_int32, POINTER(LansHParams), c_void_p, c_int64,
                                       c_void_p]),
    "rafhip_lans_plan_set_dynamic_scale": (c_int, [c_void_p, c_void_p, c_void_p]),
    "rafhip_sgd_plan_create": (c_int, [c_int32, POINTER(c_int64), c_int32, POINTER(c_void_p)]),
    "rafhip_sgd_plan_destroy": (c_int, [c_void_p]),
    "rafhip_sgd_multi_step": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                      POINTER(c_void_p), c_int32, c_double, c_double, c_void_p]),
    "rafhip_l2norm_workspace_bytes": (c_int64, [c_int64]),
    "rafhip_l2norm": (c_int, [c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_int64, c_void_p]),
    "rafhip_fuse_plan_create": (c_int, [c_int32, POINTER(c_int64), POINTER(c_void_p)]),
    "rafhip_fuse_plan_destroy": (c_int, [c_void_p]),
    "rafhip_fuse_plan_total_bytes": (c_int64, [c_void_p]),
    "rafhip_fuse_tensors": (c_int, [c_void_p, POINTER(c_void_p), c_void_p, c_void_p]),
    "rafhip_defuse_tensor": (c_int, [c_void_p, c_void_p, POINTER(c_void_p), c_void_p]),
    "rafhip_lans_read_norms": (c_int, [c_void_p, c_void_p, POINTER(c_double), c_void_p]),
    "rafhip_lans_debug_trace": (c_int, [c_void_p, POINTER(ctypes.c_uint64), c_int64, POINTER(c_int64)]),
    "rafhip_lans_timing_enable": (c_int, [c_void_p, c_int32]),
    "rafhip_lans_timing_read": (c_int, [c_void_p, c_int32, POINTER(c_float)]),
}

class TensorDesc(Structure):
    """``rafhip_tensor_desc`` of include/rafhip_dialect.h."""

    _fields_ = [
        ("data", c_void_p),
        ("device_type", c_int32),
        ("device_id", c_int32),
        ("dtype_code", c_int32),
        ("dtype_bits", c_int32),
        ("ndim", c_int32),
        ("shape", POINTER(c_int64)),
    ]


DIALECT_SYMBOLS = {
    "rafhip_raf_last_error": (c_char_p, []),
    "rafhip_raf_dispatch_list": (c_int, [c_char_p, c_int32, c_char_p, c_int32]),
    "rafhip_raf_set_dialect_preference": (c_int, [c_char_p]),
    "rafhip_raf_sgd_make": (c_int, [POINTER(TensorDesc), POINTER(TensorDesc), POINTER(TensorDesc),
                                    c_double, c_double, POINTER(c_void_p)]),
    "rafhip_raf_sgd_execute": (c_int, [c_void_p] + [POINTER(TensorDesc)] * 5 + [c_void_p]),
    "rafhip_raf_lans_make": (c_int, [c_int32, POINTER(TensorDesc), POINTER(TensorDesc), c_float,
                                     c_float, c_float, c_float, c_int32, c_float, c_int32, c_int32,
                                     c_int32, POINTER(c_void_p)]),
    "rafhip_raf_lans_mixed_make": (c_int, [c_int32, POINTER(TensorDesc), POINTER(TensorDesc), c_float,
                                     c_float, c_float, c_float, c_int32, c_float, c_int32, c_int32,
                                     c_int32, POINTER(c_void_p)]),
    "rafhip_raf_lans_execute": (c_int, [c_void_p, c_int32, POINTER(TensorDesc),
                                        POINTER(TensorDesc), c_void_p, c_int64, c_void_p]),
    "rafhip_raf_tuple_make": (c_int, [c_int32, POINTER(TensorDesc), POINTER(c_void_p)]),
    "rafhip_raf_tuple_replace": (c_int, [c_void_p, c_int32, c_int32, POINTER(TensorDesc), POINTER(c_void_p)]),
    "rafhip_raf_tuple_rebind": (c_int, [c_void_p, c_int32, c_int32, POINTER(TensorDesc), POINTER(c_int32)]),
    "rafhip_raf_tuple_size": (c_int32, [c_void_p]),
    "rafhip_raf_tuple_destroy": (c_int, [c_void_p]),
    "rafhip_raf_lans_execute_tuple": (c_int, [c_void_p, c_void_p, POINTER(TensorDesc), c_void_p, c_int64,
                                              c_void_p, c_int32]),
    "rafhip_raf_sgd_multi_execute_tuple": (c_int, [c_void_p, c_void_p, c_void_p, c_int32]),
    "rafhip_raf_sgd_multi_make": (c_int, [c_int32, c_int32, POINTER(TensorDesc), c_double, c_double,
                                          POINTER(c_void_p)]),
    "rafhip_raf_sgd_multi_execute": (c_int, [c_void_p, c_int32, POINTER(TensorDesc), c_void_p]),
    "rafhip_raf_l2norm_make": (c_int, [POINTER(TensorDesc), POINTER(c_void_p)]),
    "rafhip_raf_l2norm_execute": (c_int, [c_void_p, POINTER(TensorDesc), POINTER(TensorDesc), c_void_p,
                                          c_int64, c_void_p]),
    "rafhip_raf_fuse_tensor_make": (c_int, [c_int32, POINTER(TensorDesc), POINTER(c_void_p)]),
    "rafhip_raf_fuse_tensor_execute": (c_int, [c_void_p, c_int32, POINTER(TensorDesc), POINTER(TensorDesc),
                                               c_void_p]),
    "rafhip_raf_defuse_tensor_make": (c_int, [POINTER(TensorDesc), c_int32, POINTER(c_int64), c_int32,
                                              POINTER(c_int64), c_int32, POINTER(c_int64), POINTER(c_void_p)]),
    "rafhip_raf_defuse_tensor_execute": (c_int, [c_void_p, POINTER(TensorDesc), c_int32, POINTER(TensorDesc),
                                                 c_void_p]),
    "rafhip_raf_serve_stream_requests": (c_int, [c_int32]),
    "rafhip_raf_env_num_outputs": (c_int32, [c_void_p]),
    "rafhip_raf_env_output": (c_int, [c_void_p, c_int32, POINTER(c_int32), POINTER(c_int32), POINTER(c_int32),
                                      POINTER(c_int64), c_int32]),
    "rafhip_raf_device_count": (c_int, [c_int32, POINTER(c_int32)]),
    "rafhip_raf_device_copy": (c_int, [POINTER(TensorDesc), POINTER(TensorDesc), c_void_p]),
    "rafhip_raf_stream_create": (c_int, [c_int32, c_int32, POINTER(c_void_p)]),
    "rafhip_raf_stream_free": (c_int, [c_int32, c_int32, c_void_p]),
    "rafhip_raf_event_create": (c_int, [c_int32, c_int32, ctypes.c_uint32, POINTER(c_void_p)]),
    "rafhip_raf_event_free": (c_int, [c_int32, c_int32, c_void_p]),
    "rafhip_raf_event_record": (c_int, [c_int32, c_void_p, c_void_p]),
    "rafhip_raf_event_elapsed_ms": (c_int, [c_int32, c_void_p, c_void_p, POINTER(c_float)]),
    "rafhip_raf_stream_wait_event": (c_int, [c_int32, c_void_p, c_void_p]),
    "rafhip_raf_wait": (c_int, [c_int32, c_int32, c_int32, c_void_p]),
    "rafhip_raf_memory_alloc": (c_int, [c_int32, c_int32, c_int64, c_int64, c_int32, c_void_p, POINTER(c_void_p)]),
    "rafhip_raf_memory_data": (c_void_p, [c_void_p]),
    "rafhip_raf_memory_free": (c_int, [c_void_p]),
    "rafhip_raf_pool_init": (c_int, [c_int32, c_int32, c_char_p]),
    "rafhip_raf_pool_remove": (c_int, [c_int32, c_int32]),
    "rafhip_raf_pool_reset": (c_int, [c_int32, c_int32]),
    "rafhip_raf_pool_info": (c_int, [c_int32, c_int32, c_char_p, c_int32, POINTER(c_float), POINTER(c_float)]),
    "rafhip_raf_pool_alloc_bytes": (c_int64, [c_int32, c_int32, c_int64]),
    "rafhip_raf_env_workspace_bytes": (c_int64, [c_void_p]),
    "rafhip_raf_traced_sgd_make": (c_int, [POINTER(TensorDesc), POINTER(TensorDesc), POINTER(TensorDesc),
                                           c_double, c_double, POINTER(c_void_p)]),
    "rafhip_raf_traced_sgd_execute": (c_int, [c_void_p] + [POINTER(TensorDesc)] * 3 + [c_void_p]),
    "rafhip_raf_env_ir_text": (c_int, [c_void_p, c_int32, c_char_p, c_int32]),
    "rafhip_raf_traced_optimizer_make": (c_int, [c_int32, c_int32] + [POINTER(TensorDesc)] * 6 +
                                         [c_int32, POINTER(c_double), c_int32, c_int32, POINTER(c_void_p)]),
    "rafhip_raf_traced_optimizer_execute": (c_int, [c_void_p, c_int32] + [POINTER(TensorDesc)] * 6 +
                                            [c_int32, c_void_p, c_int64, c_void_p]),
    "rafhip_raf_env_graph_ops": (c_int, [c_void_p, c_char_p, c_int32]),
    "rafhip_raf_env_set_learning_rate": (c_int, [c_void_p, c_double]),
    "rafhip_raf_env_set_grad_unscale": (c_int, [c_void_p, c_float]),
    "rafhip_raf_env_set_dynamic_scale": (c_int, [c_void_p, POINTER(TensorDesc), POINTER(TensorDesc)]),
    "rafhip_raf_env_name": (c_char_p, [c_void_p]),
    "rafhip_raf_env_op": (c_char_p, [c_void_p]),
    "rafhip_raf_env_destroy": (c_int, [c_void_p]),
}

# include/rafhip_device.h: the HIP runtime calls behind the rocm DeviceAPI (same library)
DEVICE_SYMBOLS = {
    "rafhip_dev_set": (c_int, [c_int32]),
    "rafhip_dev_alloc": (c_int, [c_int64, POINTER(c_void_p)]),
    "rafhip_dev_free": (c_int, [c_void_p]),
    "rafhip_dev_alloc_async": (c_int, [c_int32, c_int64, c_void_p, POINTER(c_void_p)]),
    "rafhip_dev_free_async": (c_int, [c_void_p, c_void_p]),
    "rafhip_dev_pool_size": (c_int, [c_int32, POINTER(c_int64), POINTER(c_int64)]),
    "rafhip_dev_memcpy": (c_int, [c_void_p, c_void_p, c_int64, c_int32, c_void_p]),
    "rafhip_dev_memcpy_peer": (c_int, [c_void_p, c_int32, c_void_p, c_int32, c_int64, c_void_p]),
    "rafhip_dev_stream_create": (c_int, [c_int32, POINTER(c_void_p)]),
    "rafhip_dev_stream_destroy": (c_int, [c_int32, c_void_p]),
    "rafhip_dev_event_create": (c_int, [c_int32, ctypes.c_uint32, POINTER(c_void_p)]),
    "rafhip_dev_event_destroy": (c_int, [c_int32, c_void_p]),
    "rafhip_dev_event_elapsed_ms": (c_int, [c_void_p, c_void_p, POINTER(c_float)]),
    "rafhip_dev_event_record": (c_int, [c_void_p, c_void_p]),
    "rafhip_dev_stream_wait_event": (c_int, [c_void_p, c_void_p]),
    "rafhip_dev_sync_device": (c_int, [c_int32]),
    "rafhip_dev_sync_stream": (c_int, [c_void_p]),
    "rafhip_dev_sync_event": (c_int, [c_void_p]),
}

_optim = None
_dialect = None
_glue = None


def _bind(lib, table):
    for name, (restype, argtypes) in table.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes


def optim():
    """The kernel library, loaded once."""
    global _optim
    if _optim is None:
        if not OPTIM_LIB.exists():
            raise RuntimeError(
                f"{OPTIM_LIB} is missing: build it with `python -m raf_amd.build` "
                "(hipcc --offload-arch=gfx950); there is no fallback path")
        lib = ctypes.CDLL(str(OPTIM_LIB), mode=ctypes.RTLD_GLOBAL)
        _bind(lib, OPTIM_SYMBOLS)
        _bind(lib, DEVICE_SYMBOLS)
        _optim = lib
    return _optim


def last_error() -> str:
    return optim().rafhip_last_error().decode("utf-8", "replace")


def check(status: int) -> None:
    if status != RAFHIP_OK:
        raise RafHipError(status, last_error())


def dialect():
    """The C++ host layer (OpEnv / dialect registry mirror + the `hip` dialect), loaded once."""
    global _dialect
    if _dialect is None:
        optim()  # dependency, resolved through RTLD_GLOBAL / rpath
        if not DIALECT_LIB.exists():
            raise RuntimeError(
                f"{DIALECT_LIB} is missing: build it with `python -m raf_amd.build`")
        lib = ctypes.CDLL(str(DIALECT_LIB), mode=ctypes.RTLD_GLOBAL)
        _bind(lib, DIALECT_SYMBOLS)
        _dialect = lib
    return _dialect


def glue():
    """The CPython module that reads lists of torch tensors for the operator front end."""
    global _glue
    if _glue is None:
        if not GLUE_LIB.exists():
            raise RuntimeError(f"{GLUE_LIB} is missing: build it with `python -m raf_amd.build`")
        import importlib.machinery
        import importlib.util

        import torch  # noqa: F401  (the module resolves its symbols in torch's libraries)

        loader = importlib.machinery.ExtensionFileLoader("_torch_glue", str(GLUE_LIB))
        spec = importlib.util.spec_from_loader("_torch_glue", loader)
        module = importlib.util.module_from_spec(spec)
        loader.exec_module(module)
        _glue = module
    return _glue


class RafError(RuntimeError):
    """The host layer raised (the reference would surface a TVMError from dmlc::Error)."""


def check_raf(status: int) -> None:
    if status != 0:
        raise RafError(dialect().rafhip_raf_last_error().decode("utf-8", "replace"))

"""ctypes binding of libmi355x_kmeans.so (declared in include/mi355x_kmeans.h).

The library is the only compute path of this package: if it is missing, importing this
module raises (there is no CPU or PyTorch fallback).  torch tensors are used strictly as
device buffers: `ptr(t)` hands their address to the C ABI.
"""

import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_int32, c_int64, c_size_t, c_void_p

import numpy as np

# torch ships its own copy of the HIP runtime.  It has to be in the process before this
# library is loaded, so that both bind to the same runtime: with the load order reversed the
# process holds two runtimes and the second one finds no device.
import torch  # noqa: F401  (imported for its side effect on the loader)

KMX_F32 = 0
KMX_F64 = 1

KMX_RUNNING = 0
KMX_CONVERGED_STRICT = 1
KMX_CONVERGED_TOL = 2
KMX_MAX_ITER = 3
KMX_NEED_RELOCATION = 4

# kmeans++ samplers (KMX_KPP_SAMPLER_* of the header)
KMX_KPP_SAMPLER_SCAN = 0
KMX_KPP_SAMPLER_LITERAL = 1

KMX_ERR_BAD_PLAN = -7

# kernel selection flags (KMX_FLAG_* of the header)
FLAG_PATH_STREAM = 0x1
FLAG_PATH_REGISTER = 0x2
FLAG_PATH_MFMA = 0x3
FLAG_PATH_GEMM = 0x4
FLAG_LABELS_F32 = 0x10
FLAG_LABELS_SCREEN = 0x20


def flag_wgs_per_cu(x):
    return (int(x) & 0xF) << 8


def flag_cols(x):
    return (int(x) & 0x7) << 12


ABI_VERSION = 3

LIB_NAME = "libmi355x_kmeans.so"
# (KMX_LIBRARY_PATH: another build of the same library, for experiments; read when this module is imported)
LIB_PATH = os.environ.get("KMX_LIBRARY_PATH") or os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)


class LloydStatus(ctypes.Structure):
    """Mirror of kmx_lloyd_status."""

    _fields_ = [
        ("n_iter", c_int32),
        ("state", c_int32),
        ("n_empty", c_int32),
        ("n_changed", ctypes.c_uint32),
        ("shift_sum", c_double),
        ("tol", c_double),
        ("max_iter", c_int32),
        ("ticket", ctypes.c_uint32),
        ("max_sq_dist", c_double),
        ("reserved", c_int64 * 2),
    ]


assert ctypes.sizeof(LloydStatus) == 64


class LloydPlan(ctypes.Structure):
    """Mirror of kmx_lloyd_plan: shape, flags, chosen kernel variant, workspace size."""

    _fields_ = [
        ("magic", ctypes.c_uint32),
        ("abi_version", c_int32),
        ("n", c_int64),
        ("d", c_int32),
        ("k", c_int32),
        ("dtype", c_int32),
        ("flags", ctypes.c_uint32),
        ("variant", c_int32),
        ("reserved", c_int32),
        ("workspace_bytes", ctypes.c_uint64),
        ("check", ctypes.c_uint64),
    ]


assert ctypes.sizeof(LloydPlan) == 56

_P = c_void_p
_I32 = c_int32
_I64 = c_int64
_SZ = c_size_t
_U32 = ctypes.c_uint32
_PLAN = POINTER(LloydPlan)

# name -> (restype, argtypes); must list every function of include/mi355x_kmeans.h
SIGNATURES = {
    "kmx_abi_version": (_I32, []),
    "kmx_error_string": (c_char_p, [_I32]),
    "kmx_lloyd_plan_init": (_I32, [_PLAN, _I64, _I32, _I32, _I32, _U32]),
    "kmx_lloyd_workspace_bytes": (_SZ, [_I64, _I32, _I32, _I32, _U32]),
    "kmx_lloyd_init": (_I32, [_PLAN, _P, _SZ, _P, _P, _P, _I32, c_double, _P]),
    "kmx_lloyd_iter": (_I32, [_PLAN, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "kmx_lloyd_iter_traced": (_I32, [_PLAN, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "kmx_lloyd_trace_collect": (_I32, [_P, _P, _P]),
    "kmx_lloyd_iter_timed": (_I32, [_PLAN, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P,
                                    POINTER(ctypes.c_float)]),
    "kmx_lloyd_finalize": (_I32, [_PLAN, _P, _P, _P, _P, _SZ, _P]),
    "kmx_lloyd_status_read": (_I32, [_P, POINTER(LloydStatus), _P]),
    "kmx_lloyd_recheck_count": (_I32, [_PLAN, _P, POINTER(ctypes.c_uint32), _P]),
    "kmx_screen_scores": (_I32, [_P, _P, _P, _P, _P, _P, _P, _I64, _I32, _I32, _P]),
    "kmx_lloyd_kernel_variant": (_I32, [_I64, _I32, _I32, _I32, _U32]),
    "kmx_lloyd_plan_reads_rowmajor": (_I32, [_PLAN]),
    "kmx_assign_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "kmx_assign_workspace_bytes_for": (_SZ, [_I64, _I32, _I32, _I32, _U32]),
    "kmx_assign_labels": (_I32, [_P, _P, _P, _P, _SZ, _I64, _I32, _I32, _I32, _U32, _P]),
    "kmx_per_sample_inertia": (_I32, [_P, _P, _P, _P, _P, _I64, _I32, _I32, _I32, _P]),
    "kmx_inertia_workspace_bytes": (_SZ, [_I64]),
    "kmx_inertia": (_I32, [_P, _P, _P, _P, _P, _P, _SZ, _I64, _I32, _I32, _I32, _P]),
    "kmx_assign_inertia_workspace_bytes": (_SZ, [_I64, _I32, _I32, _I32, _U32]),
    "kmx_assign_labels_inertia": (_I32, [_P, _P, _P, _P, _P, _P, _SZ, _I64, _I32, _I32, _I32, _U32, _P]),
    "kmx_euclidean_distances": (_I32, [_P, _P, _P, _I64, _I32, _I32, _I32, _P]),
    "kmx_relocate_empty_clusters": (_I32, [_P, _P, _P, _P, _P, _I32, _P, _P, _P, _I64, _I32, _I32, _I32, _P]),
    "kmx_rng_init_states": (_I32, [ctypes.c_uint64, _I32, _I32, _P]),
    "kmx_rng_next_raw": (_I32, [_P, _I32, _I32, _P]),
    "kmx_kpp_workspace_bytes": (_SZ, [_I64, _I32, _I32, _I32, _I32]),
    "kmx_kpp_init": (_I32, [_P, _P, _I32, _P, _P, _P, _SZ, _I64, _I32, _I32, _I32, _I32, _U32, _P]),
    "kmx_kpp_sample_candidates": (_I32, [_P, _P, _P, _P, _SZ, _I64, _I32, _I32, _I32, _I32, _U32, _P]),
    "kmx_kpp_step": (_I32, [_P, _P, _I32, _P, _P, _P, _SZ, _I64, _I32, _I32, _I32, _I32, _U32, _P]),
    "kmx_kpp_run": (_I32, [_P, _P, _P, _I32, _P, _P, _P, _SZ, _I64, _I32, _I32, _I32, _I32, _U32, _P]),
    "kmx_kpp_closest_ptr": (_P, [_P, _I64, _I32, _I32, _I32, _I32]),
    "kmx_kpp_potentials_ptr": (_P, [_P, _I64, _I32, _I32, _I32, _I32]),
    "kmx_kpp_candidates_ptr": (_P, [_P, _I64, _I32, _I32, _I32, _I32]),
    "kmx_sum_workspace_bytes": (_SZ, [_I64, _I64]),
    "kmx_sum_rows": (_I32, [_P, _P, _I64, _I64, _I32, _P, _SZ, _I32, _P]),
    "kmx_sum_rows_static": (_I32, [_P, _P, _I64, _I64, _I32, _I32, _P]),
    "kmx_sum_cols": (_I32, [_P, _P, _I64, _I64, _P, _SZ, _I32, _P]),
    "kmx_argmin": (_I32, [_P, _P, _I64, _I32, _P]),
    "kmx_half_sq_norms": (_I32, [_P, _P, _I32, _I32, _I32, _P]),
    "kmx_broadcast_rows": (_I32, [_P, _P, _I64, _I64, _I32, _I32, _P]),
    "kmx_broadcast_div_cols": (_I32, [_P, _P, _I64, _I64, _I32, _P]),
    "kmx_divide_by": (_I32, [_P, _I64, c_double, _I32, _P]),
    "kmx_transpose": (_I32, [_P, _P, _I64, _I64, _I32, _P]),
    "kmx_fill_zero": (_I32, [_P, _I64, _P]),
    "kmx_centroid_shifts": (_I32, [_P, _P, _P, _I32, _I32, _I32, _P]),
    "kmx_topk_workspace_bytes": (_SZ, [_I64, _I32]),
    "kmx_topk_rows_workspace_bytes": (_SZ, [_I64, _I64, _I32, _I32]),
    "kmx_topk_idx": (_I32, [_P, _P, _I64, _I32, _P, _SZ, _I32, _P]),
    "kmx_topk_idx_rows": (_I32, [_P, _P, _I64, _I64, _I32, _P, _SZ, _I32, _P]),
    "kmx_topk_values": (_I32, [_P, _P, _I64, _I64, _I32, _P, _SZ, _I32, _P]),
    "kmx_is_same_clustering": (_I32, [_P, _P, _P, _P, _I64, _I32, _P]),
    "kmx_count_distinct_clusters": (_I32, [_P, _P, _P, _I64, _I32, _P]),
    "kmx_matmul": (_I32, [_P, _P, _P, _I32, _I32, _I32, _I32, _P]),
    "kmx_matmul_fused": (_I32, [_P, _P, _P, _I32, _I32, _I32, _I32, _I32, c_double, _I32, _P]),
    "kmx_probe_copy": (_I32, [_P, _P, _SZ, _P]),
    "kmx_probe_read": (_I32, [_P, _SZ, _P, _P]),
    "kmx_probe_mfma": (_I32, [_I32, _I32, _P, POINTER(c_double), _P]),
    "kmx_probe_issue": (_I32, [_I32, _I32, _I32, _P, _P]),
}


class KmxError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        super().__init__(f"{where} failed with code {code}: {error_string(code)}")


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python sklearn-numba-dpex_amd/_build.py` "
            "(hipcc, gfx950).  This engine has no fallback path."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.kmx_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_NAME} has ABI {lib.kmx_abi_version()}, expected {ABI_VERSION}")
    return lib


lib = _load()


def error_string(code):
    return lib.kmx_error_string(int(code)).decode()


def check(code, where):
    if code != 0:
        raise KmxError(code, where)


def _flags_from_environment():
    """Kernel selection for callers that pass no flags, from KMX_LLOYD_ASSIGN = f32 | screen,
    KMX_LLOYD_VARIANT = stream | register | mfma, KMX_LLOYD_WGS_PER_CU = 1..8 and
    KMX_LLOYD_COLS = 2 | 4.  Read ONCE, when this module is imported: the library itself never
    looks at the environment, and later changes of these variables have no effect."""
    flags = 0
    flags |= {"f32": FLAG_LABELS_F32, "screen": FLAG_LABELS_SCREEN}.get(os.environ.get("KMX_LLOYD_ASSIGN", ""), 0)
    flags |= {"stream": FLAG_PATH_STREAM, "register": FLAG_PATH_REGISTER,
              "mfma": FLAG_PATH_MFMA, "gemm": FLAG_PATH_GEMM}.get(os.environ.get("KMX_LLOYD_VARIANT", ""), 0)
    wgs = os.environ.get("KMX_LLOYD_WGS_PER_CU", "")
    if wgs.isdigit() and 1 <= int(wgs) <= 8:
        flags |= flag_wgs_per_cu(int(wgs))
    cols = os.environ.get("KMX_LLOYD_COLS", "")
    if cols in ("2", "4"):
        flags |= flag_cols(int(cols))
    return flags


DEFAULT_FLAGS = _flags_from_environment()


def lloyd_plan(n, d, k, dtype_code_, flags=None):
    """A filled kmx_lloyd_plan (flags=None: the import-time defaults)."""
    plan = LloydPlan()
    check(lib.kmx_lloyd_plan_init(ctypes.byref(plan), int(n), int(d), int(k), int(dtype_code_),
                                  DEFAULT_FLAGS if flags is None else int(flags)), "kmx_lloyd_plan_init")
    return plan


def dtype_code(dtype):
    dtype = np.dtype(dtype) if not hasattr(dtype, "is_floating_point") else dtype
    name = str(dtype).replace("torch.", "")
    if name == "float32":
        return KMX_F32
    if name == "float64":
        return KMX_F64
    raise ValueError(f"unsupported dtype {dtype}; expected float32 or float64")


def ptr(tensor):
    """Device address of a torch tensor (None -> NULL).  The tensor must be contiguous."""
    if tensor is None:
        return None
    if not tensor.is_contiguous():
        raise ValueError("device buffers handed to the C ABI must be contiguous")
    return tensor.data_ptr()


def current_stream():
    import torch

    return torch.cuda.current_stream().cuda_stream

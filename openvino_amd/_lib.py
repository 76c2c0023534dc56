"""ctypes binding of the C ABI declared in include/ovfcc.h and include/ovfcc_graph.h (libovfcc.so) and of the
benchmark helpers declared in include/ovfcc_bench.h (libovfcc_bench.so)."""
from __future__ import annotations

import ctypes
import os

PKG = os.path.dirname(os.path.abspath(__file__))
# OVFCC_LIB_DIR: a directory with another build of the two libraries (experiments); default: beside this file
LIB_DIR = os.environ.get("OVFCC_LIB_DIR") or PKG
LIB_PATH = os.path.join(LIB_DIR, "libovfcc.so")
BENCH_LIB_PATH = os.path.join(LIB_DIR, "libovfcc_bench.so")

OK, EINVAL, EUNSUPPORTED, EDEVICE, ENOMEM = 0, -1, -2, -3, -4
NONE, U4, I4, U8, I8, F16, F32 = range(7)
TYPE = {"none": NONE, "u4": U4, "i4": I4, "u8": U8, "i8": I8, "f16": F16, "f32": F32}
KERNEL_AUTO, KERNEL_PLAIN, KERNEL_DECODE, KERNEL_PREFILL = range(4)
GLU = {None: 0, "none": 0, "swish": 1, "gelu": 2, "gelu_tanh": 3}      # OVFCC_GLU_*
GLU_GATE_SECOND = 4
DYNQUANT_I8 = 8                                                        # OVFCC_DYNQUANT_I8
W_INPUT_MAJOR = 16
DYNQUANT_PER_GROUP = 32                                                # OVFCC_DYNQUANT_PER_GROUP                                                     # OVFCC_W_INPUT_MAJOR
DYNQUANT_ASYM = 64                                                      # OVFCC_DYNQUANT_ASYM

# every symbol include/ovfcc_bench.h declares (libovfcc_bench.so)
BENCH_SYMBOLS = ["ovfcc_bench_layers", "ovfcc_bench_grouped", "ovfcc_bench_copy", "ovfcc_bench_floor", "ovfcc_bench_mfma", "ovfcc_bench_issue"]

# every symbol include/ovfcc.h and include/ovfcc_graph.h declare (libovfcc.so)
SYMBOLS = [
    "ovfcc_init", "ovfcc_destroy", "ovfcc_device_count", "ovfcc_device_mem_info", "ovfcc_weights_create", "ovfcc_weights_clone", "ovfcc_weights_concat", "ovfcc_weights_glu", "ovfcc_weights_mlp", "ovfcc_weights_export_size", "ovfcc_weights_export", "ovfcc_weights_import", "ovfcc_weights_destroy",
    "ovfcc_weights_device_bytes", "ovfcc_weights_is_tiled", "ovfcc_request_create", "ovfcc_request_destroy",
    "ovfcc_fc_run", "ovfcc_fc_run_device", "ovfcc_fc_run_device_static", "ovfcc_fc_run_grouped_device", "ovfcc_grouped_matmul_device", "ovfcc_grouped_matmul_offsets_device", "ovfcc_gather_matmul_device", "ovfcc_gather_matmul_routed_device", "ovfcc_moe_device", "ovfcc_moe_routed_device", "ovfcc_request_sync", "ovfcc_request_force_kernel",
    "ovfcc_last_kernel_info", "ovfcc_device_malloc", "ovfcc_device_free",
    "ovfcc_memcpy_h2d", "ovfcc_memcpy_d2h", "ovfcc_memcpy_d2d", "ovfcc_desc_validate", "ovfcc_env_reload", "ovfcc_tiled_sizes",
    "ovfcc_repack_host", "ovfcc_unrepack_host", "ovfcc_unpack_u4", "ovfcc_unpack_i4", "ovfcc_last_error",
    "ovfcc_version", "ovfcc_fold_match", "ovfcc_fold_model", "ovfcc_fold_gather_matmul", "ovfcc_fold_grouped_matmul", "ovfcc_fold_moe", "ovfcc_fold_weights_create", "ovfcc_fold_expert_weights_create",
]


class GroupItem(ctypes.Structure):
    """struct ovfcc_group_item"""
    _fields_ = [("weights", ctypes.c_void_p), ("x_dev", ctypes.c_void_p), ("y_dev", ctypes.c_void_p),
                ("M", ctypes.c_int64)]


class FcDesc(ctypes.Structure):
    _fields_ = [
        ("N", ctypes.c_int64), ("K", ctypes.c_int64), ("group_size", ctypes.c_int64),
        ("w_type", ctypes.c_int32), ("scale_type", ctypes.c_int32), ("zp_type", ctypes.c_int32),
        ("zp_scalar", ctypes.c_int32), ("bias_type", ctypes.c_int32), ("act_type", ctypes.c_int32),
        ("out_type", ctypes.c_int32), ("flags", ctypes.c_int32),
    ]


MAX_RANK = 6
TYPE_OTHER = 7
OP = {"other": 0, "parameter": 1, "constant": 2, "convert": 3, "subtract": 4, "multiply": 5, "reshape": 6,
      "transpose": 7, "matmul": 8, "fully_connected": 9, "add": 10, "swish": 11, "gelu": 12, "result": 13,
      "gather_matmul": 14, "gather_matmul_compressed": 15, "unsqueeze": 16, "slice": 17, "reduce_sum": 18,
      "grouped_matmul": 19, "grouped_matmul_compressed": 20}
MAX_INPUTS = 6
FUSED_SINGLE, FUSED_CONCAT, FUSED_GLU, FUSED_MLP = 0, 1, 2, 3


class GNode(ctypes.Structure):
    """struct ovfcc_gnode (include/ovfcc_graph.h)"""
    _fields_ = [("op", ctypes.c_int32), ("type", ctypes.c_int32), ("rank", ctypes.c_int32),
                ("dims", ctypes.c_int64 * MAX_RANK), ("n_inputs", ctypes.c_int32), ("inputs", ctypes.c_int32 * MAX_INPUTS),
                ("transpose_a", ctypes.c_int32), ("transpose_b", ctypes.c_int32), ("attr", ctypes.c_int32),
                ("consumers", ctypes.c_int32), ("n_ints", ctypes.c_int32), ("ints", ctypes.c_int64 * MAX_RANK)]


class Fold(ctypes.Structure):
    """struct ovfcc_fold"""
    _fields_ = [("desc", FcDesc), ("root", ctypes.c_int32), ("matmul", ctypes.c_int32), ("activations", ctypes.c_int32),
                ("weights", ctypes.c_int32), ("scales", ctypes.c_int32), ("zero_points", ctypes.c_int32),
                ("bias", ctypes.c_int32), ("scale_broadcast", ctypes.c_int32), ("zp_from_real", ctypes.c_int32),
                ("activations_f32", ctypes.c_int32), ("w_view", ctypes.c_int64 * 2), ("scale_view", ctypes.c_int64 * 2),
                ("zp_view", ctypes.c_int64 * 2), ("n_chain", ctypes.c_int32), ("chain", ctypes.c_int32 * 16)]


class GatherFold(ctypes.Structure):
    """struct ovfcc_gather_fold"""
    _fields_ = [("desc", FcDesc), ("n_experts", ctypes.c_int32), ("root", ctypes.c_int32),
                ("activations", ctypes.c_int32), ("indices", ctypes.c_int32), ("top_k", ctypes.c_int32),
                ("weights", ctypes.c_int32), ("scales", ctypes.c_int32), ("zero_points", ctypes.c_int32),
                ("bias", ctypes.c_int32), ("scale_broadcast", ctypes.c_int32), ("zp_from_real", ctypes.c_int32),
                ("bias_per_expert", ctypes.c_int32), ("activations_f32", ctypes.c_int32),
                ("w_view", ctypes.c_int64 * 3), ("scale_view", ctypes.c_int64 * 3), ("zp_view", ctypes.c_int64 * 3),
                ("n_chain", ctypes.c_int32), ("chain", ctypes.c_int32 * 16)]


class MoeFold(ctypes.Structure):
    """struct ovfcc_moe_fold"""
    _fields_ = [("gate", GatherFold), ("up", GatherFold), ("down", GatherFold), ("glu_type", ctypes.c_int32),
                ("root", ctypes.c_int32), ("hidden_states", ctypes.c_int32), ("routing", ctypes.c_int32),
                ("indices", ctypes.c_int32), ("n_chain", ctypes.c_int32), ("chain", ctypes.c_int32 * 16)]


class Fused(ctypes.Structure):
    """struct ovfcc_fused"""
    _fields_ = [("kind", ctypes.c_int32), ("n_parts", ctypes.c_int32), ("parts", ctypes.c_int32 * 4),
                ("glu_type", ctypes.c_int32), ("root", ctypes.c_int32)]


class KernelInfo(ctypes.Structure):
    _fields_ = [
        ("kernel", ctypes.c_int32), ("grid", ctypes.c_int32 * 3), ("block", ctypes.c_int32),
        ("split_k", ctypes.c_int32), ("tile_m", ctypes.c_int32), ("tile_n", ctypes.c_int32),
        ("name", ctypes.c_char * 64),
    ]


class OvfccError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"ovfcc error {code}: {message}")
        self.code = code
        self.message = message


_lib = None


def load() -> ctypes.CDLL:
    """Loads the built library; there is no fallback when it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise OvfccError(EDEVICE, f"{LIB_PATH} is not built; run python -m openvino_amd.build")
    L = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    # the benchmark helpers live in their own library; they are reached through the same object
    if os.path.exists(BENCH_LIB_PATH):
        B = ctypes.CDLL(BENCH_LIB_PATH)
        for name in BENCH_SYMBOLS:
            setattr(L, name, getattr(B, name))
    vp, i64, sz, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_size_t, ctypes.c_int
    pp = ctypes.POINTER(ctypes.c_void_p)
    sig = {
        "ovfcc_init": (ci, [ci, pp]),
        "ovfcc_destroy": (None, [vp]),
        "ovfcc_device_count": (ci, []),
        "ovfcc_weights_create": (ci, [vp, ctypes.POINTER(FcDesc), vp, vp, vp, vp, pp]),
        "ovfcc_weights_clone": (ci, [vp, pp]),
        "ovfcc_weights_concat": (ci, [pp, ci, pp]),
        "ovfcc_weights_glu": (ci, [vp, vp, ci, pp]),
        "ovfcc_weights_mlp": (ci, [vp, vp, pp]),
        "ovfcc_weights_export_size": (ci, [vp, ctypes.POINTER(ctypes.c_size_t)]),
        "ovfcc_weights_export": (ci, [vp, vp, ctypes.c_size_t]),
        "ovfcc_weights_import": (ci, [vp, vp, ctypes.c_size_t, pp]),
        "ovfcc_weights_destroy": (None, [vp]),
        "ovfcc_weights_device_bytes": (i64, [vp]),
        "ovfcc_weights_is_tiled": (ci, [vp]),
        "ovfcc_request_create": (ci, [vp, pp]),
        "ovfcc_request_destroy": (None, [vp]),
        "ovfcc_fc_run": (ci, [vp, vp, vp, vp, i64]),
        "ovfcc_fc_run_device": (ci, [vp, vp, vp, vp, i64]),
        "ovfcc_fc_run_device_static": (ci, [vp, vp, vp, vp, i64]),
        "ovfcc_fc_run_grouped_device": (ci, [vp, ctypes.POINTER(GroupItem), ci]),
        "ovfcc_grouped_matmul_device": (ci, [vp, pp, ci, vp, ctypes.POINTER(ctypes.c_int32), i64, vp]),
        "ovfcc_grouped_matmul_offsets_device": (ci, [vp, pp, ci, vp, vp, i64, vp]),
        "ovfcc_gather_matmul_device": (ci, [vp, pp, ci, vp, ci, ctypes.POINTER(ctypes.c_int32), i64, ci, vp]),
        "ovfcc_moe_device": (ci, [vp, pp, pp, ci, vp, vp, ctypes.POINTER(ctypes.c_int32), i64, ci, vp]),
        "ovfcc_gather_matmul_routed_device": (ci, [vp, pp, ci, vp, ci, vp, i64, ci, vp]),
        "ovfcc_moe_routed_device": (ci, [vp, pp, pp, ci, vp, vp, vp, i64, ci, vp]),
        "ovfcc_bench_grouped": (ci, [vp, ctypes.POINTER(GroupItem), ci, ci, ci, ctypes.POINTER(ctypes.c_float)]),
        "ovfcc_request_sync": (ci, [vp]),
        "ovfcc_request_force_kernel": (ci, [vp, ci, ci]),
        "ovfcc_last_kernel_info": (ci, [vp, ctypes.POINTER(KernelInfo)]),
        "ovfcc_bench_layers": (ci, [vp, pp, ci, vp, vp, i64, ci, ci, ci, ctypes.POINTER(ctypes.c_float)]),
        "ovfcc_device_malloc": (ci, [vp, sz, pp]),
        "ovfcc_device_mem_info": (ci, [vp, ctypes.POINTER(sz), ctypes.POINTER(sz)]),
        "ovfcc_device_free": (ci, [vp, vp]),
        "ovfcc_memcpy_h2d": (ci, [vp, vp, vp, sz]),
        "ovfcc_memcpy_d2h": (ci, [vp, vp, vp, sz]),
        "ovfcc_memcpy_d2d": (ci, [vp, vp, vp, sz]),
        "ovfcc_bench_copy": (ci, [vp, vp, vp, sz, ci, ctypes.POINTER(ctypes.c_float)]),
        "ovfcc_bench_floor": (ci, [vp, vp, sz, sz, ci, ci, ci, ci, ctypes.POINTER(ctypes.c_float)]),
        "ovfcc_bench_mfma": (ci, [vp, ci, ci, ci, ci, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_double)]),
        "ovfcc_bench_issue": (ci, [vp, ci, ci, ci, ci, ci, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
        "ovfcc_desc_validate": (ci, [ctypes.POINTER(FcDesc)]),
        "ovfcc_env_reload": (None, []),
        "ovfcc_tiled_sizes": (ci, [ctypes.POINTER(FcDesc), ctypes.POINTER(sz), ctypes.POINTER(sz), ctypes.POINTER(sz)]),
        "ovfcc_repack_host": (ci, [ctypes.POINTER(FcDesc), vp, vp, vp, vp, vp, vp]),
        "ovfcc_unrepack_host": (ci, [ctypes.POINTER(FcDesc), vp, vp, vp, vp, vp, vp]),
        "ovfcc_unpack_u4": (ci, [vp, sz, vp]),
        "ovfcc_unpack_i4": (ci, [vp, sz, vp]),
        "ovfcc_last_error": (ctypes.c_char_p, []),
        "ovfcc_version": (ctypes.c_char_p, []),
        "ovfcc_fold_match": (ci, [ctypes.POINTER(GNode), ci, ci, ctypes.POINTER(Fold)]),
        "ovfcc_fold_model": (ci, [ctypes.POINTER(GNode), ci, ctypes.POINTER(Fold), ci, ctypes.POINTER(ci),
                                  ctypes.POINTER(Fused), ci, ctypes.POINTER(ci)]),
        "ovfcc_fold_gather_matmul": (ci, [ctypes.POINTER(GNode), ci, ci, ctypes.POINTER(GatherFold)]),
        "ovfcc_fold_grouped_matmul": (ci, [ctypes.POINTER(GNode), ci, ci, ctypes.POINTER(GatherFold)]),
        "ovfcc_fold_moe": (ci, [ctypes.POINTER(GNode), ci, ci, ctypes.POINTER(MoeFold)]),
        "ovfcc_fold_weights_create": (ci, [vp, ctypes.POINTER(GNode), ci, ctypes.POINTER(Fold), ctypes.POINTER(vp), ci, pp]),
        "ovfcc_fold_expert_weights_create": (ci, [vp, ctypes.POINTER(GNode), ci, ctypes.POINTER(GatherFold), ci,
                                                  ctypes.POINTER(vp), ci, pp]),
    }
    for name, (res, args) in sig.items():
        if name in BENCH_SYMBOLS and not hasattr(L, name):
            continue
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


_env_seen = None


def sync_env() -> None:
    """The library reads its OVFCC_* overrides once; a Python host that changes os.environ afterwards (tests,
    experiments) has them read again before its next call."""
    global _env_seen
    now = tuple(sorted((k, v) for k, v in os.environ.items() if k.startswith("OVFCC_")))
    if now != _env_seen:
        if _env_seen is not None or now:
            load().ovfcc_env_reload()
        _env_seen = now


def check(rc: int) -> None:
    if rc != OK:
        raise OvfccError(rc, load().ovfcc_last_error().decode())

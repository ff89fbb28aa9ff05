"""ctypes bindings of the two in-tree shared libraries.

libmi355_backend.so  — HIP kernels behind the C ABI of include/mi355_abi.h
libmirage_runtime.so — the mirage:: C++ host API and its C facade (csrc/host/c_api.cc)

There is no fallback: if the libraries are missing the import fails, and any
device work without an MI355X aborts inside the runtime.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
BACKEND_PATH = os.path.join(_HERE, "libmi355_backend.so")
RUNTIME_PATH = os.path.join(_HERE, "libmirage_runtime.so")

MAX_OPERATORS, MAX_PARAMETERS = 16, 120


class Mi355Plan(ctypes.Structure):
    """struct mi355_plan (include/mi355_abi.h)."""
    _fields_ = [
        ("grid_dim", ctypes.c_int * 3), ("block_dim", ctypes.c_int * 3),
        ("forloop_range", ctypes.c_int), ("reduction_dimx", ctypes.c_int),
        ("smem_bytes", ctypes.c_int), ("num_operators", ctypes.c_int),
        ("num_parameters", ctypes.c_int), ("num_dmem_inputs", ctypes.c_int),
        ("num_dmem_outputs", ctypes.c_int),
        ("operator_types", ctypes.c_int * MAX_OPERATORS),
        ("parameters", ctypes.c_int * MAX_PARAMETERS),
    ]


class Mi355DeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 64),
                ("compute_units", ctypes.c_int), ("clock_mhz", ctypes.c_int),
                ("memory_clock_mhz", ctypes.c_int), ("lds_bytes_per_block", ctypes.c_int),
                ("total_memory", ctypes.c_size_t)]


class Mi355LaunchInfo(ctypes.Structure):
    _fields_ = [("kernel_id", ctypes.c_int), ("workgroups", ctypes.c_int),
                ("threads", ctypes.c_int), ("lds_bytes", ctypes.c_int),
                ("row_split", ctypes.c_int)]


class MirageCPlan(ctypes.Structure):
    """struct mirage_c_plan (csrc/host/c_api.cc)."""
    _fields_ = [
        ("grid_dim", ctypes.c_int * 3), ("block_dim", ctypes.c_int * 3),
        ("forloop_range", ctypes.c_int), ("reduction_dimx", ctypes.c_int),
        ("num_inputs", ctypes.c_int), ("input_map", (ctypes.c_int * 3) * 4),
        ("forloop_dim", ctypes.c_int * 4), ("input_smem_layout", ctypes.c_int * 4),
        ("output_map", ctypes.c_int * 3), ("num_ops", ctypes.c_int),
        ("op_type", ctypes.c_int * 16), ("op_num_operands", ctypes.c_int * 16),
        ("op_operands", ((ctypes.c_int * 2) * 2) * 16),
    ]


class MirageVerifyStats(ctypes.Structure):
    """mirage_verify_stats of csrc/host/verify.cc."""
    _fields_ = [("kernel_ops", ctypes.c_int), ("customized_ops", ctypes.c_int),
                ("compares", ctypes.c_int), ("fp_bytes", ctypes.c_longlong),
                ("matmul_macs", ctypes.c_longlong),
                ("enqueue_seconds", ctypes.c_double), ("wait_seconds", ctypes.c_double)]


# every symbol include/mi355_abi.h declares, with its signature
_vp, _ci, _sz, _u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_uint64
_pi = ctypes.POINTER(ctypes.c_int)
_pf = ctypes.POINTER(ctypes.c_float)
_pll = ctypes.POINTER(ctypes.c_longlong)
_pplan = ctypes.POINTER(Mi355Plan)
_pvp = ctypes.POINTER(ctypes.c_void_p)
ABI = {
    "mi355_init": (_ci, [_sz, _pvp]),
    "mi355_shutdown": (_ci, []),
    "mi355_is_initialised": (_ci, []),
    "mi355_last_error": (ctypes.c_char_p, []),
    "mi355_get_device_info": (_ci, [ctypes.POINTER(Mi355DeviceInfo)]),
    "mi355_set_option": (_ci, [_ci, _ci]),
    "mi355_launch_floor": (_ci, [_ci, _pf]),
    "mi355_get_tables": (_ci, [_pvp, _pvp, _pvp]),
    "mi355_memcpy_h2d": (_ci, [_vp, _vp, _sz]),
    "mi355_memcpy_d2h": (_ci, [_vp, _vp, _sz]),
    "mi355_memset": (_ci, [_vp, _ci, _sz]),
    "mi355_copy": (_ci, [_vp, _vp, _sz]),
    "mi355_sync": (_ci, []),
    "mi355_queue_select": (_ci, [_ci]),
    "mi355_fp_fill_iota": (_ci, [_vp, _sz]),
    "mi355_fp_fill_uniform": (_ci, [_vp, _sz, _u64]),
    "mi355_fp_fill_many": (_ci, [_pvp, ctypes.POINTER(_sz), ctypes.POINTER(_u64), _ci, _ci]),
    "mi355_fp_matmul": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci]),
    "mi355_fp_unary": (_ci, [_ci, _vp, _vp, _sz]),
    "mi355_fp_matmul_many": (_ci, [_pvp, _pvp, _pvp, _pi, _pi, _pi, _pi, _ci]),
    "mi355_fp_binary": (_ci, [_ci, _vp, _pi, _vp, _pi, _vp, _pi, _ci]),
    "mi355_fp_binary_many": (_ci, [_pi, _pvp, _pi, _pvp, _pi, _pvp, _pi, _pi, _ci]),
    "mi355_fp_reduce": (_ci, [_vp, _vp, _sz, _ci, _ci, _ci]),
    "mi355_fp_equal": (_ci, [_vp, _vp, _sz, _pi]),
    "mi355_fp_big_tiles_check": (_ci, [_pi]),
    "mi355_fp_equal_reset": (_ci, [_ci, _ci]),
    "mi355_fp_equal_enqueue": (_ci, [_vp, _vp, _sz, _ci]),
    "mi355_fp_equal_enqueue_many": (_ci, [_pvp, _pvp, ctypes.POINTER(_sz), _pi, _ci]),
    "mi355_fp_equal_collect": (_ci, [_ci, _ci, _vp]),
    "mi355_fp_equal_read": (_ci, [_ci, _ci, _vp]),
    "mi355_queue_current": (_ci, []),
    "mi355_mark_record": (_ci, [_ci]),
    "mi355_mark_wait_queue": (_ci, [_ci, _ci]),
    "mi355_mark_wait_host": (_ci, [_ci]),
    "mi355_customized_fp": (_ci, [_pplan, _pvp, _pvp]),
    "mi355_customized_fp_static": (_ci, [_pplan, _pvp, _pvp]),
    "mi355_customized_fp_batch": (_ci, [_pplan, _ci, _pvp, _pvp]),
    "mi355_plan_extents": (_ci, [_pplan, _pll, _pll, _pi, _pi]),
    "mi355_customized_run": (_ci, [_pplan, _pvp, _pvp]),
    "mi355_customized_profile": (_ci, [_pplan, _pvp, _pvp, _ci, _ci, _ci, _pf]),
    "mi355_last_launch": (_ci, [ctypes.POINTER(Mi355LaunchInfo)]),
    "mi355_phase_trace_read": (_ci, [ctypes.POINTER(ctypes.c_ulonglong), _sz]),
    "mi355_f16_fill_iota": (_ci, [_vp, _sz, _ci]),
    "mi355_f16_fill_normal": (_ci, [_vp, _sz, ctypes.c_float, _u64]),
    "mi355_f16_matmul": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci]),
    "mi355_f16_matmul_layout": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _ci]),
    "mi355_f16_transpose": (_ci, [_vp, _vp, _ci, _ci, _ci]),
    "mi355_f16_unary": (_ci, [_ci, _vp, _vp, _sz]),
    "mi355_f16_binary": (_ci, [_ci, _vp, _pi, _vp, _pi, _vp, _pi, _ci]),
    "mi355_f16_reduce": (_ci, [_vp, _vp, _sz, _ci, _ci, _ci]),
    "mi355_emit_hip_preamble": (ctypes.c_char_p, []),
    "mi355_emit_hip_kernel": (ctypes.c_longlong, [_pplan, ctypes.c_char_p, _ci, ctypes.c_char_p,
                                                  ctypes.c_longlong]),
    "mi355_timer_start": (_ci, []),
    "mi355_timer_stop": (_ci, [_pf]),
}

class MirageLayoutStats(ctypes.Structure):
    _fields_ = [("assignments", ctypes.c_longlong), ("measurements", ctypes.c_longlong),
                ("unrunnable", ctypes.c_longlong),
                ("truncated", ctypes.c_int), ("first_ms", ctypes.c_float),
                ("best_ms", ctypes.c_float), ("worst_ms", ctypes.c_float)]


# float cost(void *user, int op_index, int const *layouts, int n)
LAYOUT_COST_FN = ctypes.CFUNCTYPE(ctypes.c_float, ctypes.c_void_p, ctypes.c_int,
                                  ctypes.POINTER(ctypes.c_int), ctypes.c_int)

FACADE = {
    "mirage_graph_create": (_vp, []),
    "mirage_graph_destroy": (None, [_vp]),
    "mirage_graph_num_operators": (_ci, [_vp]),
    "mirage_graph_new_input": (_vp, [_vp, _pi, _ci, _ci, _ci]),
    "mirage_graph_matmul": (_vp, [_vp, _vp, _vp]),
    "mirage_graph_unary": (_vp, [_vp, _ci, _vp]),
    "mirage_graph_binary": (_vp, [_vp, _ci, _vp, _vp]),
    "mirage_graph_reduction": (_vp, [_vp, _vp, _ci, _ci]),
    "mirage_graph_customized": (_ci, [_vp, _pvp, _ci, ctypes.POINTER(MirageCPlan), _pvp, _ci]),
    "mirage_graph_pop_operator": (_ci, [_vp]),
    "mirage_op_type": (_ci, [_vp, _ci]),
    "mirage_op_num_outputs": (_ci, [_vp, _ci]),
    "mirage_op_output": (_vp, [_vp, _ci, _ci]),
    "mirage_op_fingerprint": (_ci, [_vp, _ci]),
    "mirage_op_profile": (ctypes.c_float, [_vp, _ci]),
    "mirage_op_execute": (_ci, [_vp, _ci]),
    "mirage_op_lowered": (_ci, [_vp, _ci, _ci, _pplan, _pi]),
    "mirage_tensor_info": (_ci, [_vp, _pi, _pi, _pi, _pi, _pll]),
    "mirage_tensor_ptr": (_vp, [_vp, _ci]),
    "mirage_tensor_write": (_ci, [_vp, _ci, _vp, _sz]),
    "mirage_tensor_read": (_ci, [_vp, _ci, _vp, _sz]),
    "mirage_tensor_same_fingerprint": (_ci, [_vp, _vp]),
    "mirage_graph_fingerprint": (_ci, [_vp, _u64, ctypes.POINTER(MirageVerifyStats)]),
    "mirage_verify_batch": (_ci, [_pvp, _ci, _vp, _u64, _vp, ctypes.POINTER(MirageVerifyStats)]),
    "mirage_verify_batch_begin": (_vp, [_pvp, _ci, _vp, _u64, _ci]),
    "mirage_verify_set_queues_per_batch": (None, [_ci]),
    "mirage_verify_ring_create": (_vp, []),
    "mirage_verify_ring_destroy": (None, [_vp]),
    "mirage_verify_ring_acquire": (_ci, [_vp, _ci, _pi, _pi]),
    "mirage_verify_ring_release": (None, [_vp, _ci]),
    "mirage_verify_batch_end": (_ci, [_vp, _ci, _vp, ctypes.POINTER(MirageVerifyStats)]),
    "mirage_optimize_layout": (_ci, [_vp, ctypes.c_longlong, LAYOUT_COST_FN, _vp,
                                     ctypes.POINTER(MirageLayoutStats)]),
    "mirage_graph_generate_hip_program": (_ci, [_vp, ctypes.c_char_p]),
    "mirage_graph_from_json": (_vp, [ctypes.c_char_p]),
    "mirage_graph_to_json": (ctypes.c_longlong, [_vp, ctypes.c_char_p, ctypes.c_longlong]),
    "mirage_checkpoint_load": (_vp, [ctypes.c_char_p]),
    "mirage_checkpoint_destroy": (None, [_vp]),
    "mirage_checkpoint_num_graphs": (_ci, [_vp]),
    "mirage_checkpoint_summary": (ctypes.c_float, [_vp, _pll]),
    "mirage_checkpoint_json": (ctypes.c_longlong, [_vp, _ci, ctypes.c_char_p, ctypes.c_longlong]),
    "mirage_graph_profile": (ctypes.c_float, [_vp, _pf, _ci]),
    "mirage_set_smem_budget": (None, [_sz]),
    "mirage_get_smem_budget": (_sz, []),
    "mirage_device_ready": (_ci, []),
    "mirage_arena_offset": (ctypes.c_longlong, []),
    "mirage_arena_total": (ctypes.c_longlong, []),
}

_backend = None
_runtime = None


def _bind(lib, table):
    for name, (res, args) in table.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args


def backend():
    """The device backend; raises if it has not been built."""
    global _backend
    if _backend is None:
        if not os.path.exists(BACKEND_PATH):
            raise ImportError(
                f"{BACKEND_PATH} is missing: build it with `python -m attention_superoptimizer_amd.build`")
        lib = ctypes.CDLL(BACKEND_PATH, mode=ctypes.RTLD_GLOBAL)
        _bind(lib, ABI)
        _backend = lib
    return _backend


def runtime():
    """The host runtime (loads the backend first)."""
    global _runtime
    if _runtime is None:
        backend()
        if not os.path.exists(RUNTIME_PATH):
            raise ImportError(
                f"{RUNTIME_PATH} is missing: build it with `python -m attention_superoptimizer_amd.build`")
        lib = ctypes.CDLL(RUNTIME_PATH, mode=ctypes.RTLD_GLOBAL)
        _bind(lib, FACADE)
        _runtime = lib
    return _runtime


def last_error() -> str:
    return backend().mi355_last_error().decode()

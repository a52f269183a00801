"""Loader of libseedless_hip.so (the C ABI in include/seedless_hip.h).

There is no fallback: if the library has not been built (`python -c "import __graft_entry__ as g;
g.build()"` or `make -C qwisp_amd/csrc`) importing this module raises.
"""
import ctypes as C
import os

from . import abi

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "libseedless_hip.so")

# name -> (restype, argtypes); every symbol include/seedless_hip.h declares
_i32, _i64, _u64, _f32, _vp, _sz = C.c_int32, C.c_int64, C.c_uint64, C.c_float, C.c_void_p, C.c_size_t
SIGNATURES = {
    "sl_create": (_i32, [C.POINTER(abi.ModelDesc), _i32, _i32, C.POINTER(_vp)]),
    "sl_destroy": (None, [_vp]),
    "sl_fault": (C.c_char_p, [_vp]),
    "sl_inject_failure": (None, [_vp]),
    "sl_step_argmax": (_i32, [_vp, _vp, _i32, _vp]),
    "sl_step_sample_rows": (_i32, [_vp, _vp, _i32, _f32, _f32, _u64, _vp]),
    "sl_lane_create": (_i32, [_vp, _i32, _i32, _vp]),
    "sl_lane_step_argmax": (_i32, [_vp, _i32, _vp, _vp]),
    "sl_chained_step_argmax": (_i32, [_vp, _i32, _i32, _vp]),
    "sl_forward_rows": (_i32, [_vp, _vp, _i32, _i32, _vp]),
    "sl_forward_tokens": (_i32, [_vp, _vp, _i32, _vp]),
    "sl_head_argmax_rows": (_i32, [_vp, _i32, _i32, _vp]),
    "sl_hidden_rows": (_i32, [_vp, _i32, _vp]),
    "sl_logits_row": (_i32, [_vp, _i32, _vp]),
    "sl_head_argmax": (_i32, [_vp, _vp, _i32, _vp]),
    "sl_head_argmax_noalloc": (_i32, [_vp, _vp, _i32, _vp, _vp]),
    "sl_snapshot": (_i32, [_vp, C.POINTER(abi.Snap)]),
    "sl_rollback_one_step": (_i32, [_vp, C.POINTER(abi.Snap)]),
    "sl_full_snapshot": (_i32, [_vp, C.POINTER(_vp)]),
    "sl_full_restore": (_i32, [_vp, _vp]),
    "sl_full_snap_free": (None, [_vp]),
    "sl_persist_size": (_sz, [_vp]),
    "sl_persist_write": (_i32, [_vp, _vp, _sz]),
    "sl_persist_restore": (_i32, [_vp, _vp, _sz]),
    "sl_read_layer_cache": (_i32, [_vp, _i32, _vp, _vp]),
    "sl_load_layer_cache": (_i32, [_vp, _i32, _vp, _vp, _i32]),
    "sl_position": (_i32, [_vp]),
    "sl_read_route": (_i32, [_vp, _i32, _i32, _vp, _vp]),
    "sl_moe_block_rows": (_i32, [_vp, _i32, _vp, _i32, _vp]),
    "sl_gdn_layer_rows": (_i32, [_vp, _i32, _vp, _i32, _vp]),
    "sl_attn_layer_rows": (_i32, [_vp, _i32, _vp, _i32, _vp]),
    "sl_debug_scratch": (_i32, [_vp, _i32, _vp, _sz]),
    "sl_greedy_generate": (_i32, [_vp, _vp, _i32, _i32, _i32, _vp]),
    "sl_suffix_draft": (_i32, [_vp, _i32, _i32, _i32, _i32, _vp]),
    "sl_spec_gate_threshold": (_i32, [_i32]),
    "sl_spec_gate_window_needed": (_i32, [_i32]),
    "sl_spec_gate_should_suspend": (_i32, [_vp, _i32, _i32]),
    "sl_spec_generate": (_i32, [_vp, _vp, _i32, _i32, C.POINTER(abi.SpecOptions), _vp, C.POINTER(abi.SpecStats)]),
    "sl_spec_generate_backend": (_i32, [C.POINTER(abi.SpecBackend), _vp, _i32, _i32, C.POINTER(abi.SpecOptions), _vp,
                                        C.POINTER(abi.SpecStats)]),
    "sl_sched_create": (_i32, [C.POINTER(abi.BatchSlots), _i32, abi.TOKEN_FN, abi.FINISH_FN, _vp, C.POINTER(_vp)]),
    "sl_sched_destroy": (None, [_vp]),
    "sl_sched_submit": (_i32, [_vp, _vp, _i32, _i32, _vp, _i32]),
    "sl_sched_round": (_i32, [_vp]),
    "sl_lane_slots_create": (_i32, [_vp, _i32, _i32, _i32, C.c_long, C.POINTER(_vp), C.POINTER(abi.BatchSlots)]),
    "sl_lane_slots_destroy": (None, [_vp]),
    "sl_reset": (_i32, [_vp]),
    "sl_max_rows": (_i32, [_vp]),
    "sl_last_gpu_ms": (_f32, [_vp]),
    "sl_stream": (_vp, [_vp]),
    "sl_set_persistent": (_i32, [_vp, _i32]),
    "sl_set_hybrid": (_i32, [_vp, _i32]),
    "sl_debug_stage_clock": (_i32, [_vp, _i32, _vp, _i32]),
    "sl_stage_clock_words": (_i32, []),
    "sl_debug_set_spin_limit": (_i32, [_vp, C.c_uint32]),
    "sl_debug_set_flow_counter": (_i32, [_vp, C.c_uint32]),
    "sl_debug_flow_tags": (_i32, [C.c_uint32, _i32, _i32, _i32, _i32, _vp, _vp]),
    "sl_ubench_exchange": (_i32, [_i32, _i32, C.POINTER(_f32)]),
    "sl_ubench_gemv_stream": (_i32, [_i32, _i32, C.POINTER(_f32)]),
    "sl_ubench_mfma_issue": (_i32, [_i32, _i32, _i32, C.POINTER(_f32), C.POINTER(_f32)]),
    "sl_profile_head": (_i32, [_vp, _i32]),
    "sl_profile_head_read": (_i32, [_vp, C.POINTER(C.c_double), C.POINTER(_i64)]),
    "sl_selftest_math": (_i32, [_i32, _vp, _vp, _i64]),
    "sl_selftest_qmm4": (_i32, [_vp, _i32, _vp, _vp, _vp, _i32, _i32, _vp]),
    "sl_synth_q4": (_i32, [_vp, _vp, _vp, _i64, _i32, _u64, _f32, _vp]),
    "sl_synth_f16": (_i32, [_vp, _i64, _u64, _f32, _f32, _vp]),
    "sl_synth_f32": (_i32, [_vp, _i64, _u64, _f32, _f32, _vp]),
}


class SeedlessError(RuntimeError):
    def __init__(self, what, status, fault=None):
        self.status, self.fault = status, fault
        super().__init__(f"{what} failed with status {status}" + (f": {fault}" if fault else ""))


class Library:
    def __init__(self, path=SO_PATH):
        if not os.path.exists(path):
            raise ImportError(f"{path} is not built; run __graft_entry__.build() (hipcc, gfx950). "
                              "There is no CPU fallback for the Seedless engine.")
        self.dll = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self.dll, name)       # AttributeError if the library lacks a declared symbol
            fn.restype, fn.argtypes = res, args

    @staticmethod
    def check(status, what, fault=None):
        if status != abi.SL_OK:
            raise SeedlessError(what, status, fault)


_lib = None


def get():
    global _lib
    if _lib is None:
        _lib = Library()
    return _lib

"""ctypes binding of libdifflogic_hip.so.  The library is the only implementation of the GPU
path: if it is missing or a symbol is absent, importing this module's users fails loudly."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdifflogic_hip.so")

DL_OK = 0
DL_ERR_INVALID_ARGUMENT = 1
DL_ERR_BIT_COUNT = 2
DL_ERR_NOT_DIVISIBLE = 3
DL_ERR_DTYPE = 4
DL_ERR_LAUNCH = 5
DL_ERR_TOO_LARGE = 6
DL_ERR_SCRATCH_LIMIT = 7
DL_ERR_CAPTURING = 8

DL_F16, DL_F32, DL_F64, DL_F16_W32, DL_F64_W32 = 0, 1, 2, 3, 4

DL_STATIC_SCRATCH_BYTES = 64 << 20      # include/difflogic_hip.h

_vp, _i64, _int, _dbl = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_double

# name -> argument types; every function returns int (dl_status) unless listed in _RESTYPES.
SIGNATURES = {
    "dl_version": [],
    "dl_status_string": [_int],
    "dl_last_hip_error": [],
    "dl_logic_forward": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp],
    "dl_logic_backward_w": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp],
    "dl_logic_forward_logits": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp],
    "dl_logic_backward_logits": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp],
    "dl_logic_forward_chained": [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp],
    "dl_logic_backward_w_chained": [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp],
    "dl_logic_backward_x": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _dbl, _int, _vp],
    "dl_backward_schedule_build": [_vp, _vp, _i64, _i64, _vp, _vp, _vp, ctypes.POINTER(_i64)],
    "dl_logic_backward_chained": [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _int, _vp, _vp, _i64, _i64, _vp, _vp, _vp,
                                  _i64, _i64, _i64, _dbl, _int, _vp],
    "dl_logic_forward_chained_lower": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                       _int, _vp],
    "dl_logic_backward_chained_lower": [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _int, _vp, _vp, _i64, _i64, _vp, _vp, _vp,
                                        _vp, _vp, _vp, _vp, _int, _vp, _i64, _i64, _i64, _dbl, _int, _vp],
    "dl_logic_backward_chained_workspace_bytes": [_i64, _i64, _i64, _int],
    "dl_group_sum_workspace_bytes": [_i64, _i64, _i64, _int],
    "dl_group_sum_forward": [_vp, _vp, _vp, _i64, _i64, _i64, _dbl, _int, _vp],
    "dl_group_sum_backward": [_vp, _vp, _i64, _i64, _i64, _dbl, _int, _vp],
    "dl_logic_forward_group_sum": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _dbl, _int, _vp],
    "dl_logic_backward_logits_grouped": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp],
    "dl_logic_backward_x_grouped": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _dbl, _int, _vp],
    "dl_logic_backward_chained_grouped": [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _int, _vp, _vp, _i64, _i64, _vp, _vp,
                                          _vp, _i64, _i64, _i64, _i64, _dbl, _int, _vp],
    "dl_adam_max_tensors": [],
    "dl_adam_step": [_int, _vp, _vp, _vp, _vp, _vp, _vp, _dbl, _dbl, _dbl, _dbl, _dbl, _vp],
    "dl_gate_ids": [_vp, _vp, _i64, _int, _vp],
    "dl_fold_gate_constants": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp],
    "dl_gate_ids_folded": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _i64, _vp],
    "dl_mark_live_inputs": [_vp, _vp, _vp, _vp, _vp, _i64, _vp],
    "dl_logic_eval": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp],
    "dl_tensor_packbits": [_vp, _vp, _i64, _i64, _int, ctypes.POINTER(_i64), _vp],
    "dl_tensor_packbits_batch_major": [_vp, _vp, _i64, _i64, _int, ctypes.POINTER(_i64), _vp],
    "dl_tensor_packbits_batch_major_rows": [_vp, _vp, _i64, _i64, _i64, _vp],
    "dl_groupbitsum": [_vp, _vp, _i64, _i64, _int, _i64, _i64, _vp],
    "dl_logic_eval_fused_workspace_bytes": [_int, _i64],
    "dl_logic_eval_fused": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _vp, _vp],
    "dl_eval_schedule_chunk": [],
    "dl_eval_schedule_capacity": [_i64, _int],
    "dl_eval_schedule_build": [_vp, _vp, _i64, _i64, _int, _vp, _vp, _vp],
    "dl_logic_eval_chained_workspace_bytes": [_int, _i64, _i64],
    "dl_logic_eval_chained": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _i64, _int, _vp, _vp],
    "dl_logic_eval_fused_groupbitsum_workspace_bytes": [_int, _i64, _i64, _int, _i64],
    "dl_logic_eval_fused_groupbitsum": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _i64, _i64, _vp, _vp, _vp],
    "dl_logic_eval_fused_groupbitsum_noalloc": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _i64, _i64, _vp, _vp],
    "dl_logic_net_lds_max_width": [],
    "dl_logic_net_lds_workspace_bytes": [_int, _vp],
    "dl_logic_net_lds_groupbitsum": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _i64, _i64, _vp, _vp],
    "dl_logic_net_lds_groupbitsum_scheduled": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _i64,
                                               _i64, _vp, _vp],
    "dl_logic_net_lds_groupbitsum_bool": [_vp, _i64, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp],
    "dl_logic_net_lds_groupbitsum_thinned": [_vp, _int, _i64, _int, _vp, _vp, _vp, _int, _vp, _vp, _i64, _int, _i64, _i64, _vp, _vp],
    "dl_count_chain_block": [],
    "dl_count_chain_padded_steps": [_i64],
    "dl_count_chain_plan_build": [_vp, _i64, _i64, _i64, _vp, _vp, ctypes.POINTER(_int)],
    "dl_logic_eval_chained_groupbitsum_workspace_bytes": [_i64, _int, _i64, _int, _i64],
    "dl_logic_eval_chained_groupbitsum": [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _i64, _int, _vp,
                                          _i64, _int, _i64, _i64, _vp, _vp],
    "dl_count_group": [],
    "dl_count_order_build": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp],
}
_RESTYPES = {"dl_status_string": ctypes.c_char_p, "dl_last_hip_error": ctypes.c_char_p, "dl_group_sum_workspace_bytes": ctypes.c_int64,
             "dl_logic_eval_fused_workspace_bytes": ctypes.c_int64,
             "dl_eval_schedule_capacity": ctypes.c_int64, "dl_eval_schedule_build": ctypes.c_int64,
             "dl_backward_schedule_build": ctypes.c_int64,
             "dl_logic_backward_chained_workspace_bytes": ctypes.c_int64,
             "dl_logic_eval_fused_groupbitsum_workspace_bytes": ctypes.c_int64,
             "dl_logic_eval_chained_workspace_bytes": ctypes.c_int64,
             "dl_count_chain_padded_steps": ctypes.c_int64, "dl_count_chain_plan_build": ctypes.c_int64,
             "dl_logic_eval_chained_groupbitsum_workspace_bytes": ctypes.c_int64,
             "dl_logic_net_lds_max_width": ctypes.c_int64, "dl_logic_net_lds_workspace_bytes": ctypes.c_int64}

_lib = None


def load():
    """Loads the library once and declares every prototype of include/difflogic_hip.h."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP kernel library has not been built. "
            "Run `python difflogic_amd/build.py` (needs hipcc); there is no fallback implementation.")
    # torch first: its own copy of the HIP runtime must be the one in the process when the library's
    # dependency on libamdhip64 is resolved.  Loaded the other way round, the process ends up with
    # two runtimes and every launch from this library fails with "no ROCm-capable device".
    import torch  # noqa: F401
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, ctypes.c_int)
    _lib = lib
    return lib


def status_string(status: int) -> str:
    text = load().dl_status_string(int(status)).decode()
    if int(status) == DL_ERR_LAUNCH:
        text += f" ({load().dl_last_hip_error().decode()})"
    return text

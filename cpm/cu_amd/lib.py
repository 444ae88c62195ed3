"""ctypes binding of ``libcpmcu_amd.so`` (the C-ABI declared in ``include/cpmcu_amd.h``).

Loading fails loudly when the library has not been built: there is no fallback implementation.
torch is imported first so that the library binds to the HIP runtime torch already loaded
(one runtime per process: streams and device pointers are shared with torch).
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime this library must share)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcpmcu_amd.so")

OK, ERR_INVALID_ARGUMENT, ERR_RUNTIME, ERR_UNSUPPORTED, ERR_HIP = range(5)

c_int, c_float, c_size_t = ctypes.c_int, ctypes.c_float, ctypes.c_size_t
c_void_p, c_char_p, c_u64 = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_uint64
_P = c_void_p

# name -> (restype, argtypes); status-returning functions are wrapped to raise
SIGNATURES = {
    "cpmcu_last_error": (c_char_p, []),
    "cpmcu_version": (c_char_p, []),
    "cpmcu_set_option": (c_int, [c_char_p, c_int]),
    "cpmcu_init_base_model": (c_int, [c_float, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_float, c_float, c_float]),
    "cpmcu_init_eagle_model": (c_int, [c_int] * 5),
    "cpmcu_init_minicpm4_eagle_model": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int]),
    "cpmcu_init_storage": (c_int, [ctypes.POINTER(c_int)]),
    "cpmcu_load_model": (c_int, [c_char_p, c_u64]),
    "cpmcu_prefill": (c_int, [c_int, c_int, c_u64, c_u64, c_u64]),
    "cpmcu_decode": (c_int, [c_int, c_int, c_u64, c_u64, c_u64, c_u64, c_u64, c_int]),
    "cpmcu_draft": (c_int, [c_u64] * 5),
    "cpmcu_verify_and_fix": (c_int, [c_int, c_u64, c_u64, c_u64, c_u64, c_u64, c_u64, ctypes.POINTER(c_int)]),
    "cpmcu_verify_step": (c_int, [c_int, c_int, c_int, _P, _P, _P, _P] + [c_u64] * 13 + [c_int, c_int]),
    "cpmcu_capture_begin": (c_int, []),
    "cpmcu_capture_end": (c_int, [ctypes.POINTER(c_int)]),
    "cpmcu_graph_replay": (c_int, [c_int]),
    "cpmcu_graph_destroy": (c_int, [c_int]),
    "cpmcu_step_graph_count": (c_int, []),
    "cpmcu_print_perf_summary": (c_int, []),
    "cpmcu_decode_attention": (c_int, [c_int, c_int, c_int, c_u64, c_u64, c_u64, c_u64, c_u64, c_u64]),
    "cpmcu_draft_attention": (c_int, [c_int, c_int, c_int, c_u64, c_u64, c_u64, c_u64, c_u64, c_int, c_u64]),
    "cpmcu_decode_lm_head": (c_int, [c_int, c_u64, c_u64, c_u64]),
    "cpmcu_draft_head": (c_int, [c_int, c_u64, c_u64, c_u64, c_u64]),
    "cpmcu_draft_round": (c_int, [c_int, c_u64, c_u64, c_u64, c_u64]),
    "cpmcu_draft_finish": (c_int, [c_u64] * 5),
    "cpmcu_set_block_table": (c_int, [_P, c_int]),
    "cpmcu_model_pointers": (c_int, [c_int, ctypes.POINTER(c_u64), ctypes.POINTER(c_u64), ctypes.POINTER(c_u64), ctypes.POINTER(c_int)]),
    "cpmcu_stream": (c_u64, []),
    "cpmcu_synchronize": (c_int, []),
    "cpmcu_attention_abandoned_waits": (ctypes.c_long, []),
    "cpmcu_shutdown": (c_int, []),
    "cpmcu_kv_append": (c_int, [_P, _P, _P, _P, _P, _P, c_int, c_int, _P]),
    "cpmcu_tree_attention_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "cpmcu_tree_attention": (c_int, [_P, _P, _P, _P, _P, c_int, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_float, _P, _P, c_size_t, c_int, _P]),
    "cpmcu_tree_attention_rope": (c_int, [_P, _P, _P, _P, _P, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_float, _P, _P, c_size_t, c_int, _P]),
    "cpmcu_tree_attention_window": (c_int, [_P, _P, _P, _P, _P, c_int, _P, _P, _P, c_int, _P, c_int, c_int, c_int, c_int, c_int, c_float, _P, _P, c_size_t, c_int, _P]),
    "cpmcu_tree_attention_merge_mode": (c_int, [_P]),
    "cpmcu_tree_attention_release_workspace": (c_int, [_P]),
    "cpmcu_frspec_head_mode": (c_int, [_P, c_int, c_int, c_int, c_int, c_int]),
    "cpmcu_head_release_workspace": (c_int, [_P]),
    "cpmcu_frspec_fused_rows": (c_int, [ctypes.POINTER(ctypes.c_long), ctypes.POINTER(ctypes.c_long), ctypes.POINTER(ctypes.c_long)]),
    "cpmcu_tree_attention_plan": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_char_p, c_size_t, ctypes.POINTER(c_int), ctypes.POINTER(c_int), ctypes.POINTER(c_int)]),
    "cpmcu_rope_table": (c_int, [_P, _P, c_int, _P, _P]),
    "cpmcu_rope_apply": (c_int, [_P, c_int, c_int, c_int, _P, _P, _P]),
    "cpmcu_gather_rows": (c_int, [_P, _P, c_int, c_int, _P, _P]),
    "cpmcu_head_workspace_bytes": (c_size_t, [c_int, c_int]),
    "cpmcu_head_weight_tiled_bytes": (c_size_t, [c_int, c_int]),
    "cpmcu_head_weight_tile": (c_int, [_P, _P, c_int, c_int, _P, _P]),
    "cpmcu_frspec_head_topk": (c_int, [_P, _P, c_int, _P, c_int, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, c_size_t, _P]),
    "cpmcu_lm_head_argmax": (c_int, [_P, _P, c_int, c_int, c_int, c_int, c_int, c_float, _P, _P, _P, c_size_t, _P]),
    "cpmcu_head_plan": (c_int, [c_int, c_int, c_int, c_int, c_char_p, c_size_t, ctypes.POINTER(c_int)]),
    "cpmcu_lm_head_partials": (c_int, [_P, _P, c_int, c_int, c_int, c_int, c_int, c_float, _P, _P, c_size_t, ctypes.POINTER(c_int), ctypes.POINTER(c_int), _P]),
    "cpmcu_lm_head_argmax_static_scratch_bytes": (c_size_t, []),
    "cpmcu_lm_head_argmax_static": (c_int, [_P, _P, c_int, c_int, c_int, c_int, c_int, c_float, _P, _P, _P]),
    "cpmcu_log_softmax": (c_int, [_P, c_int, c_int, _P, _P]),
    "cpmcu_topk_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "cpmcu_topk": (c_int, [_P, c_int, c_int, c_int, _P, _P, _P, c_size_t, _P]),
    "cpmcu_remap": (c_int, [_P, c_int, _P, _P, _P]),
    "cpmcu_tree_accept": (c_int, [c_int, _P, _P, _P, _P, _P, c_int, _P, _P, _P]),
    "cpmcu_kv_compact": (c_int, [_P, _P, c_int, _P, c_int, _P, _P, _P, _P, c_int, _P]),
    "cpmcu_accept_commit": (c_int, [_P, _P, c_int, _P, c_int, _P, _P, _P, _P, _P, c_int, _P, c_int, _P, _P, _P, c_int, _P]),
    "cpmcu_verify_tail": (c_int, [_P, _P, c_int, _P, c_int, c_int, _P, _P, _P, c_int, c_int, _P, _P, _P, c_int, _P, _P, c_int, _P, _P, _P, _P, _P, _P, _P, _P]),
    "cpmcu_verify_tail_inplace": (c_int, [_P, _P, c_int, _P, _P, _P, _P, c_int, _P]),
    "cpmcu_draft_tree_state_bytes": (c_size_t, [c_int, c_int]),
    "cpmcu_draft_tree_begin": (c_int, [_P, c_int, c_int, _P, _P, _P, _P, _P, _P]),
    "cpmcu_draft_tree_extend": (c_int, [_P, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P]),
    "cpmcu_draft_tree_finish": (c_int, [_P, c_int, c_int, c_int, _P, _P, _P, _P, _P, _P, _P]),
}


def load_raw():
    """The bare ctypes library with argtypes/restypes set (no exception wrapping)."""
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libcpmcu_amd.so is not built (expected at %s); run `python -m cpm.cu_amd.build`. "
            "There is no fallback implementation." % LIB_PATH)
    raw = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(raw, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    return raw


class CpmcuLib:
    """Attribute access returns the C function without the ``cpmcu_`` prefix; status codes raise."""

    def __init__(self):
        self.raw = load_raw()

    def last_error(self):
        return self.raw.cpmcu_last_error().decode()

    def check(self, rc):
        if rc == OK:
            return
        msg = self.last_error()
        if rc == ERR_INVALID_ARGUMENT:
            raise ValueError(msg)
        raise RuntimeError(msg)

    def __getattr__(self, name):
        fn = getattr(self.raw, "cpmcu_" + name)
        if fn.restype is not c_int or name in ():
            return fn

        def call(*args):
            self.check(fn(*args))

        call.__name__ = name
        setattr(self, name, call)
        return call


_lib = None


def get():
    global _lib
    if _lib is None:
        _lib = CpmcuLib()
    return _lib

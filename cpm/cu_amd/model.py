"""The model-level side of the library from Python: the process-global model of ``libcpmcu_amd.so`` (the mirror
of the reference's pybind module, src/entry.cu:98-534) with its library-owned paged cache, heads and HIP graphs.

torch is used for two things only: the step's input/output buffers (the caller's, as in cpmcu/llm.py) and views
onto the library's pools for harnesses that fill or inspect the cache directly.
"""
import ctypes

import numpy as np
import torch

from . import lib as _libmod
from .kvcache import HEAD_DIM, PAGE, PagedKVCache


class _DeviceMemory:
    """A raw device address as an object torch can wrap without copying."""

    def __init__(self, ptr, shape, typestr):
        self.__cuda_array_interface__ = {"shape": tuple(shape), "typestr": typestr, "data": (int(ptr), False), "version": 2}


def device_view(ptr, shape, dtype=torch.float16):
    typestr = {torch.float16: "<f2", torch.int32: "<i4", torch.uint8: "|u1"}[dtype]
    return torch.as_tensor(_DeviceMemory(ptr, shape, typestr), device="cuda")


class PathModel:
    """init_base_model -> init_minicpm4_eagle_model -> init_storage -> load_model, then verify steps.

    One per process (the library keeps one global model, like the reference); ``close()`` frees it."""

    def __init__(self, vocab, layers, hidden, q_heads, kv_heads, memory_limit, scale_lmhead=1.0, frspec_vocab=0,
                 tree_size=60, num_iter=6, topk=10, draft_layers=1, eagle_window=1024, dtype=0):
        self.L = _libmod.get()
        self.vocab, self.layers, self.hidden, self.q_heads, self.kv_heads = vocab, layers, hidden, q_heads, kv_heads
        self.tree_size = tree_size
        L = self.L
        # dtype: 0 = fp16, 1 = bf16 (tensors then hold bfloat16 patterns, whatever 16-bit torch dtype carries them)
        L.init_base_model(ctypes.c_float(memory_limit), vocab, layers, hidden, 4 * hidden, q_heads, kv_heads, HEAD_DIM,
                          ctypes.c_float(1e-5), int(dtype), 2048, ctypes.c_float(1.0), ctypes.c_float(scale_lmhead), ctypes.c_float(1.0))
        # the drafter builds trees of up to 64 nodes (src/model/minicpm4/minicpm4_eagle.cuh:69); a wider tree for verify_step is the caller's
        L.init_minicpm4_eagle_model(draft_layers, num_iter, topk, min(tree_size, 64), int(dtype), 0, 128, eagle_window, frspec_vocab,
                                    ctypes.c_float(1.0), 1, 1)
        ctx = ctypes.c_int(0)
        L.init_storage(ctypes.byref(ctx))
        self.max_context = ctx.value
        kp, vp, bt, npg = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_int()
        self._k, self._v = [], []
        for l in range(layers + draft_layers):
            L.model_pointers(l, ctypes.byref(kp), ctypes.byref(vp), ctypes.byref(bt), ctypes.byref(npg))
            self._k.append(device_view(kp.value, (npg.value, kv_heads, PAGE, HEAD_DIM)))
            self._v.append(device_view(vp.value, (npg.value, kv_heads, HEAD_DIM, PAGE)))
        self.num_pages = npg.value
        self.block_table = device_view(bt.value, (npg.value,), torch.int32)

    def load_head(self, w, token_id_remap=None):
        """w: numpy fp16 [vocab, hidden] on the host (load_model copies from host pointers, src/entry.cu:466-468)."""
        if token_id_remap is not None:
            remap = np.ascontiguousarray(token_id_remap, np.int32)
            self.L.load_model(b"eagle.token_id_remap", remap.ctypes.data)
        w = np.ascontiguousarray(w, np.float16)
        self.L.load_model(b"lm_head.weight", w.ctypes.data)

    def cache(self, block_table=None, num_layers=None):
        """The library's pools of the first num_layers layers (default: the target model's) as a PagedKVCache, seen
        through `block_table` (a device int32 tensor; default: the model's own table)."""
        n = self.layers if num_layers is None else num_layers
        return PagedKVCache.from_pools(self._k[:n], self._v[:n], self.block_table if block_table is None else block_table)

    def verify_step(self, num_tokens, padded_length, q, k_new, v_new, attn_out, hidden, draft_ids, position_ids, cache_length,
                    kv_length, attn_mask, tree_parent, accepted_ids, gt_out=None, prev_hidden=None, next_position_ids=None,
                    result=None, block_table=None, advance_length=False, cuda_graph=True):
        """Enqueue one verify step on the library's stream (cpmcu_verify_step); per-layer lists of tensors."""
        arr = lambda ts: (ctypes.c_uint64 * len(ts))(*[t.data_ptr() for t in ts])
        p = lambda t: 0 if t is None else t.data_ptr()
        self.L.verify_step(len(q), num_tokens, padded_length, arr(q), arr(k_new), arr(v_new), arr(attn_out), p(hidden), p(draft_ids),
                           p(position_ids), p(cache_length), p(kv_length), p(attn_mask), p(tree_parent), p(block_table), p(gt_out),
                           p(accepted_ids), p(prev_hidden), p(next_position_ids), p(result), 1 if advance_length else 0,
                           1 if cuda_graph else 0)

    def draft_round(self, d, hidden, next_ids, parent_rows=None, draft_mask=None):
        """Round d of draft() without the dense layers (cpmcu_draft_round); tensors are the caller's static buffers."""
        p = lambda t: 0 if t is None else t.data_ptr()
        self.L.draft_round(int(d), p(hidden), p(next_ids), p(parent_rows), p(draft_mask))

    def draft_finish(self, tree_draft_ids, tree_position_ids, cache_length, tree_attn_mask, tree_parent):
        self.L.draft_finish(tree_draft_ids.data_ptr(), tree_position_ids.data_ptr(), cache_length.data_ptr(), tree_attn_mask.data_ptr(),
                            tree_parent.data_ptr())

    def draft_attention(self, draft_layer, n, padded_length, q, k_new, v_new, cache_length, mask, mask_k_range, out):
        self.L.draft_attention(int(draft_layer), int(n), int(padded_length), q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(),
                               cache_length.data_ptr(), 0 if mask is None else mask.data_ptr(), int(mask_k_range), out.data_ptr())

    def set_block_table(self, table):
        """Install a logical -> physical page table (a full permutation of the model's pages, or a prefix of one whose
        remaining pages follow in ascending order); `table`: int32 tensor or array."""
        t = np.ascontiguousarray(table.cpu().numpy() if hasattr(table, "cpu") else table, np.int32)
        self.L.set_block_table(t.ctypes.data_as(ctypes.c_void_p), t.size)

    def capture(self, fn):
        """Record the model-level calls fn() makes into a library-owned graph; returns its id for replay()."""
        self.L.capture_begin()
        try:
            fn()
        finally:
            gid = ctypes.c_int(-1)
            self.L.capture_end(ctypes.byref(gid))
        return gid.value

    def replay(self, graph_id):
        self.L.graph_replay(int(graph_id))

    def stream(self):
        """The library's stream as a torch stream object (events recorded on it time the library's launches)."""
        return torch.cuda.ExternalStream(self.L.raw.cpmcu_stream())

    def synchronize(self):
        self.L.synchronize()

    def close(self):
        self._k, self._v, self.block_table = [], [], None
        self.L.shutdown()

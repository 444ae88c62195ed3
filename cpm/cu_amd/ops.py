"""The operators of the verify/draft path on torch device tensors.

torch only supplies device memory and the current stream; every function here is a thin call into
``libcpmcu_amd.so`` through the C-ABI (``include/cpmcu_amd.h``).  Nothing falls back to torch math.
"""
import ctypes
import math

import torch

from . import lib as _libmod
from .kvcache import HEAD_DIM


def _lib():
    return _libmod.get()


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensor required"
    return ctypes.c_void_p(t.data_ptr())


def _ptr_result(t):
    """Like _ptr, but a pinned host tensor may stand in: the GPU writes it through the mapped address."""
    if t is None:
        return None
    assert (t.is_cuda or t.is_pinned()) and t.is_contiguous(), "device-resident or pinned contiguous tensor required"
    return ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


_workspaces = {}


def _workspace(kind, nbytes, device):
    key = (kind, device)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None and kind == "attn":
            release_attention_workspace(ws)
        if ws is not None and kind == "head":
            release_head_workspace(ws)
        ws = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def release_attention_workspace(ws):
    """Before an attention workspace tensor is dropped: the library gives its merge counters to another workspace.
    The device is synchronised first (no launch on the workspace may be in flight)."""
    torch.cuda.synchronize()
    _lib().tree_attention_release_workspace(ctypes.c_void_p(ws.data_ptr()))


def release_head_workspace(ws):
    """Before a head workspace tensor is dropped: the library takes back the states its one-launch FR-Spec head
    publishes through.  The device is synchronised first (no launch on the workspace may be in flight)."""
    torch.cuda.synchronize()
    _lib().head_release_workspace(ctypes.c_void_p(ws.data_ptr()))


def mask_words(T):
    return (T + 63) // 64


def kv_append(cache, layer, k_new, v_new, kv_len):
    """copy_to_kvcache (src/model/attn.cuh:14-21): rows go to positions [*kv_len - T, *kv_len)."""
    T = k_new.shape[0]
    assert k_new.dtype == torch.float16 and v_new.dtype == torch.float16 and kv_len.dtype == torch.int32
    assert k_new.numel() == T * cache.Hkv * HEAD_DIM and v_new.numel() == k_new.numel()
    _lib().kv_append(_ptr(cache.k[layer]), _ptr(cache.v[layer]), _ptr(cache.block_table), _ptr(k_new), _ptr(v_new),
                     _ptr(kv_len), T, cache.Hkv, _stream())


def rope_table(position_ids, inv_freq):
    """(cos, sin) of float(position) * inv_freq for every tree row: [T, 64, 2] fp32 (src/model/rotary.cuh:11-17)."""
    T = position_ids.numel()
    assert position_ids.dtype == torch.int32 and inv_freq.dtype == torch.float32 and inv_freq.numel() == HEAD_DIM // 2
    out = torch.empty((T, HEAD_DIM // 2, 2), dtype=torch.float32, device=position_ids.device)
    _lib().rope_table(_ptr(position_ids), _ptr(inv_freq), T, _ptr(out), _stream())
    return out


def rope_apply_(table, q, k):
    """In-place rotary embedding of q [T,Hq,128] and k [T,Hkv,128] (rotary_embedding_kernel, src/model/rotary.cuh:7-34)."""
    T, Hq, D = q.shape
    assert D == HEAD_DIM and k.shape[0] == T and k.shape[2] == D and table.shape[0] == T
    _lib().rope_apply(_ptr(table), T, Hq, k.shape[1], _ptr(q), _ptr(k), _stream())


def tree_attention(q, cache, layer, kv_len, max_kv_len, mask=None, scale=None, num_splits=0, out=None,
                   k_new=None, v_new=None, mask_k_range=0, rope=None, block_window_size=0):
    """mha_fwd_kvcache with a tree mask (src/flash_attn/flash_api.hpp:292-392) on the paged cache.

    q [T, Hq, 128] fp16; kv_len int32[1] on the device = P + T; mask uint64 [T, W] or None (chain).
    k_new / v_new [T, Hkv, 128]: the tree rows' K/V; when given the kernel appends them to the cache
    itself (src/model/attn.cuh:200) instead of expecting them there.
    mask_k_range (0 = T): number of trailing keys the mask bits refer to; k*d for the drafter's layers.
    rope [T, 64, 2] fp32 from rope_table: q and k_new are taken unrotated and rotated inside the kernel.
    block_window_size (0 = none, else >= 128 tokens): the drafter layer's block sliding window
    (src/flash_attn/src/flash_blockmask.h:32): key blocks of 128 below ceil(P/128) - window/128 are skipped.
    """
    T, Hq, D = q.shape
    assert D == HEAD_DIM and q.dtype == torch.float16 and kv_len.dtype == torch.int32
    if out is None:
        out = torch.empty_like(q)
    W = 0
    if mask is not None:
        assert mask.dtype in (torch.uint64, torch.int64)
        mask = mask.reshape(T, -1)
        W = mask.shape[1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    need = _lib().raw.cpmcu_tree_attention_workspace_bytes(T, Hq, cache.Hkv, int(max_kv_len))
    ws = _workspace("attn", need, q.device)
    if k_new is not None:
        assert k_new.dtype == torch.float16 and v_new.dtype == torch.float16
        assert k_new.numel() == T * cache.Hkv * HEAD_DIM and v_new.numel() == k_new.numel()
    if rope is not None:
        assert rope.dtype == torch.float32 and rope.numel() == T * HEAD_DIM
    if block_window_size:
        _lib().tree_attention_window(_ptr(q), _ptr(cache.k[layer]), _ptr(cache.v[layer]), _ptr(cache.block_table), _ptr(kv_len),
                                     int(max_kv_len), _ptr(k_new), _ptr(v_new), _ptr(rope), int(block_window_size), _ptr(mask), W,
                                     int(mask_k_range), T, Hq, cache.Hkv, ctypes.c_float(scale), _ptr(out), _ptr(ws), ws.numel(),
                                     int(num_splits), _stream())
        return out
    if rope is not None:
        # rotary embedding of q and of the appended K rows fused into the kernel (table from rope_table)
        _lib().tree_attention_rope(_ptr(q), _ptr(cache.k[layer]), _ptr(cache.v[layer]), _ptr(cache.block_table), _ptr(kv_len),
                                   int(max_kv_len), _ptr(k_new), _ptr(v_new), _ptr(rope), _ptr(mask), W, int(mask_k_range), T, Hq,
                                   cache.Hkv, ctypes.c_float(scale), _ptr(out), _ptr(ws), ws.numel(), int(num_splits), _stream())
        return out
    _lib().tree_attention(_ptr(q), _ptr(cache.k[layer]), _ptr(cache.v[layer]), _ptr(cache.block_table), _ptr(kv_len),
                          int(max_kv_len), _ptr(k_new), _ptr(v_new), _ptr(mask), W, int(mask_k_range), T, Hq, cache.Hkv,
                          ctypes.c_float(scale), _ptr(out),
                          _ptr(ws), ws.numel(), int(num_splits), _stream())
    return out


def gather_rows(src, remap):
    """remap_copy (src/model/tree_drafter.cuh:79-86): dst[r] = src[remap[r]]."""
    assert src.dtype == torch.float16 and remap.dtype == torch.int32
    dst = torch.empty((remap.numel(), src.shape[1]), dtype=torch.float16, device=src.device)
    _lib().gather_rows(_ptr(src), _ptr(remap), remap.numel(), src.shape[1], _ptr(dst), _stream())
    return dst


W_ROW_MAJOR, W_TILED = 0, 1
COMMIT_ADVANCE_LENGTH = 1
COMMIT_NEXT_ROOT = 2


class TiledWeight:
    """A head weight matrix in MFMA operand order (CPMCU_W_TILED): built once, streamed ~20 % faster."""

    def __init__(self, data, V, H):
        self.data, self.V, self.H = data, int(V), int(H)
        self.shape = (self.V, self.H)


def tile_head_weight(w, row_remap=None):
    """[*, H] row-major fp16 -> TiledWeight of V rows; with row_remap (int32 [V]) row r is w[row_remap[r]]
    (remap_copy, src/model/tree_drafter.cuh:79-86, fused with the re-tiling)."""
    assert w.dtype == torch.float16 and w.is_contiguous()
    H = w.shape[1]
    V = w.shape[0] if row_remap is None else row_remap.numel()
    out = torch.empty(_lib().raw.cpmcu_head_weight_tiled_bytes(V, H) // 2, dtype=torch.float16, device=w.device)
    _lib().head_weight_tile(_ptr(w), _ptr(row_remap), V, H, _ptr(out), _stream())
    return TiledWeight(out, V, H)


def _weight(w):
    if isinstance(w, TiledWeight):
        return w.data, W_TILED, w.V
    return w, W_ROW_MAJOR, w.shape[0]


def frspec_head_topk(hidden, w, token_id_remap, k):
    """FR-Spec draft head: logits -> log-softmax -> top-k -> full-vocabulary ids.

    Returns dict(logits [n,V] f16 raw, row_stats [n,2] f32 (max, ln sum), val [n,k] f16, pos [n,k] i32, ids [n,k] i32).
    """
    n, H = hidden.shape
    w, layout, V = _weight(w)
    dev = hidden.device
    logits = torch.empty((n, V), dtype=torch.float16, device=dev)
    stats = torch.empty((n, 2), dtype=torch.float32, device=dev)
    val = torch.empty((n, k), dtype=torch.float16, device=dev)
    pos = torch.empty((n, k), dtype=torch.int32, device=dev)
    ids = torch.empty((n, k), dtype=torch.int32, device=dev)
    ws = _workspace("head", _lib().raw.cpmcu_head_workspace_bytes(n, V), dev)
    _lib().frspec_head_topk(_ptr(hidden), _ptr(w), layout, _ptr(token_id_remap), n, V, H, k, _ptr(logits), _ptr(stats),
                            _ptr(val), _ptr(pos), _ptr(ids), _ptr(ws), ws.numel(), _stream())
    return dict(logits=logits, row_stats=stats, val=val, pos=pos, ids=ids)


def frspec_head_plan(n, w, k):
    """Kernel name(s) of a frspec_head_topk call with n hidden rows on matrix w: the one-launch kernel when the shape
    allows it and the library has a publication state for the head workspace, else GEMM + top-k."""
    w_, layout, V = _weight(w)
    H = w.H if isinstance(w, TiledWeight) else w.shape[1]
    gemm = head_plan(n, w)[0]
    ws = _workspace("head", _lib().raw.cpmcu_head_workspace_bytes(n, V), w_.device)
    if _lib().raw.cpmcu_frspec_head_mode(ctypes.c_void_p(ws.data_ptr()), layout, n, V, H, k) == 1:
        nb, fp, kc = gemm[gemm.index("<") + 1:-1].split(",")
        return "frspec_head_topk_kernel<%s,%s>" % (fp, kc)
    # the row kernel: on the whole row up to 32768 elements, on slices of it beyond
    return gemm + ("+topk_row_kernel<true>" if V <= 32768 else "+topk_row_kernel<true>+topk_slice_merge_kernel<true>")


def lm_head_argmax(hidden, w, head_scale=None, want_logits=False, gt=None):
    """Target head + arg-max (src/model/linear.cuh:82-101 + torch argmax of tree_drafter.py:233)."""
    n, H = hidden.shape
    w, layout, V = _weight(w)
    dev = hidden.device
    logits = torch.empty((n, V), dtype=torch.float16, device=dev) if want_logits else None
    if gt is None:
        gt = torch.empty(n, dtype=torch.int32, device=dev)
    ws = _workspace("head", _lib().raw.cpmcu_head_workspace_bytes(n, V), dev)
    _lib().lm_head_argmax(_ptr(hidden), _ptr(w), layout, n, V, H, 0 if head_scale is None else 1,
                          ctypes.c_float(1.0 if head_scale is None else head_scale), _ptr(logits), _ptr(gt),
                          _ptr(ws), ws.numel(), _stream())
    return (gt, logits) if want_logits else gt


class HeadPartials:
    """The target head's arg-max left as per-workgroup partials (cpmcu_lm_head_partials): finished by verify_tail."""

    def __init__(self, workspace, num_partials, stride, n):
        self.workspace, self.num_partials, self.stride, self.n = workspace, int(num_partials), int(stride), int(n)


def lm_head_partials(hidden, w, head_scale=None, logits=None):
    """The target head's GEMM without the launch that finishes its arg-max; see verify_tail."""
    n, H = hidden.shape
    w, layout, V = _weight(w)
    ws = _workspace("head", _lib().raw.cpmcu_head_workspace_bytes(n, V), hidden.device)
    num, stride = ctypes.c_int(0), ctypes.c_int(0)
    _lib().lm_head_partials(_ptr(hidden), _ptr(w), layout, n, V, H, 0 if head_scale is None else 1,
                            ctypes.c_float(1.0 if head_scale is None else head_scale), _ptr(logits), _ptr(ws), ws.numel(),
                            ctypes.byref(num), ctypes.byref(stride), _stream())
    return HeadPartials(ws, num.value, stride.value, n)


def verify_tail(cache, draft_ids, gt, position_ids, cache_length, attn_mask, tree_parent, hidden=None, prev_hidden=None,
                gt_out=None, best=None, path=None, accepted_ids=None, next_position_ids=None, result=None):
    """The whole tail of verify() in one launch (src/model/minicpm4/minicpm4_eagle.cuh:398-418): arg-max finish
    when `gt` is a HeadPartials, acceptance, compaction of every layer, accepted ids, hidden-row gather.
    draft_ids is read only; results go to best (a, node), path [T], accepted_ids [T], gt_out [T], ..."""
    T = draft_ids.numel()
    W = attn_mask.numel() // T
    parts = gt if isinstance(gt, HeadPartials) else None
    hidden_dim = 0 if hidden is None else hidden.shape[-1]
    _lib().verify_tail(_ptr(cache.k_ptrs), _ptr(cache.v_ptrs), cache.num_layers, _ptr(cache.block_table), cache.Hkv, T,
                       _ptr(draft_ids), None if parts else _ptr(gt), _ptr(parts.workspace) if parts else None,
                       parts.num_partials if parts else 0, parts.stride if parts else 0, _ptr(position_ids), _ptr(cache_length),
                       _ptr(attn_mask), W, _ptr(tree_parent), _ptr(hidden), hidden_dim, _ptr(prev_hidden), _ptr(gt_out), _ptr(best),
                       _ptr(path), _ptr(accepted_ids), _ptr(next_position_ids), _ptr_result(result), _stream())


def verify_tail_inplace(best, accepted_ids, pred=None, cache_length=None, kv_len=None, position_ids=None, advance_length=False,
                        next_root=False):
    """The in-place updates behind verify_tail: pred[:a] <- ids (or pred[0] <- last id), lengths and positions += a."""
    flags = (COMMIT_ADVANCE_LENGTH if advance_length else 0) | (COMMIT_NEXT_ROOT if next_root else 0)
    _lib().verify_tail_inplace(_ptr(best), _ptr(accepted_ids), accepted_ids.numel(), _ptr(pred), _ptr(cache_length), _ptr(kv_len),
                               _ptr(position_ids), flags, _stream())


def log_softmax_(x):
    """In place (src/model/eagle.cuh:29-89); returns row_stats [n,2] (max, ln sum)."""
    n, dim = x.shape
    stats = torch.empty((n, 2), dtype=torch.float32, device=x.device)
    _lib().log_softmax(_ptr(x), n, dim, _ptr(stats), _stream())
    return stats


def topk(x, top):
    """TopK::prefill (src/model/topk.cuh:255-288): value descending, ties -> lower index."""
    n, dim = x.shape
    val = torch.empty((n, top), dtype=torch.float16, device=x.device)
    pos = torch.empty((n, top), dtype=torch.int32, device=x.device)
    ws = _workspace("topk", _lib().raw.cpmcu_topk_workspace_bytes(n, dim, top), x.device)
    _lib().topk(_ptr(x), n, dim, top, _ptr(val), _ptr(pos), _ptr(ws), ws.numel(), _stream())
    return val, pos


def remap(pos, token_id_remap):
    out = torch.empty_like(pos)
    _lib().remap(_ptr(pos), pos.numel(), _ptr(token_id_remap), _ptr(out), _stream())
    return out


def tree_accept(pred, gt, position_ids, cache_length, attn_mask, tree_parent, best=None):
    """verify_kernel (src/model/tree_drafter.cuh:5-46). pred is overwritten with the path; returns best[2]."""
    T = pred.numel()
    if best is None:
        best = torch.empty(2, dtype=torch.int32, device=pred.device)
    W = attn_mask.numel() // T
    _lib().tree_accept(T, _ptr(pred), _ptr(gt), _ptr(position_ids), _ptr(cache_length), _ptr(attn_mask), W,
                       _ptr(tree_parent), _ptr(best), _stream())
    return best


def kv_compact(cache, pred, gt, cache_length, best, max_accept):
    """fix_kv_cache (src/model/tree_drafter.cuh:48-77) on every layer of the paged cache."""
    _lib().kv_compact(_ptr(cache.k_ptrs), _ptr(cache.v_ptrs), cache.num_layers, _ptr(cache.block_table), cache.Hkv,
                      _ptr(pred), _ptr(gt), _ptr(cache_length), _ptr(best), int(max_accept), _stream())


def accept_commit(cache, pred, gt, cache_length, best, max_accept, hidden=None, prev_hidden=None,
                  next_position_ids=None, result=None, advance_length=False, next_root=False, kv_len=None):
    """The rest of verify() after the acceptance (src/model/minicpm4/minicpm4_eagle.cuh:398-418): compaction,
    accepted ids, gather of the accepted hidden rows, next position ids, packed (a, ids) result and the
    device-side advance of cache_length, in two launches with the accept length staying on the device."""
    flags = (COMMIT_ADVANCE_LENGTH if advance_length else 0) | (COMMIT_NEXT_ROOT if next_root else 0)
    hidden_dim = 0 if hidden is None else hidden.shape[-1]
    _lib().accept_commit(_ptr(cache.k_ptrs), _ptr(cache.v_ptrs), cache.num_layers, _ptr(cache.block_table), cache.Hkv,
                         _ptr(pred), _ptr(gt), _ptr(cache_length), _ptr(kv_len), _ptr(best), int(max_accept), _ptr(hidden), hidden_dim,
                         _ptr(prev_hidden), _ptr(next_position_ids), _ptr_result(result), flags, _stream())


class DraftTree:
    """Tree bookkeeping of the drafter (src/model/minicpm4/minicpm4_eagle.cuh:319-393) on the device.

    One object per draft model; ``begin`` / ``extend`` / ``finish`` are one kernel each and never
    synchronise, so a whole draft can be enqueued (or graph-captured) without a host round trip.
    """

    def __init__(self, k, num_iter, token_id_remap=None, device="cuda"):
        self.k, self.num_iter = int(k), int(num_iter)
        self.remap = token_id_remap
        nbytes = _lib().raw.cpmcu_draft_tree_state_bytes(self.k, self.num_iter)
        self.state = torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=device)
        self.next_ids = torch.empty(self.k, dtype=torch.int32, device=device)
        self.parent_rows = torch.empty(self.k, dtype=torch.int32, device=device)
        self.draft_mask = torch.empty(self.k, dtype=torch.int64, device=device)

    def begin(self, topk_val, topk_pos):
        """topk_val fp16[k], topk_pos int32[k] (first row). Returns next_ids [k]."""
        assert topk_val.dtype == torch.float16 and topk_pos.dtype == torch.int32 and topk_val.numel() == self.k
        _lib().draft_tree_begin(_ptr(self.state), self.k, self.num_iter, _ptr(topk_val), _ptr(topk_pos), _ptr(self.remap),
                                _ptr(self.next_ids), _ptr(self.draft_mask), _stream())
        return self.next_ids

    def extend(self, d, topk_val, topk_pos):
        """topk_val fp16[k,k] (cumulated in place), topk_pos int32[k,k] of iteration d >= 1.
        Returns (next_ids [k], parent_rows [k], draft_mask [k])."""
        assert topk_val.dtype == torch.float16 and topk_pos.dtype == torch.int32 and topk_val.numel() == self.k * self.k
        _lib().draft_tree_extend(_ptr(self.state), self.k, self.num_iter, int(d), _ptr(topk_val), _ptr(topk_pos), _ptr(self.remap),
                                 _ptr(self.next_ids), _ptr(self.parent_rows), _ptr(self.draft_mask), _stream())
        return self.next_ids, self.parent_rows, self.draft_mask

    def finish(self, tree_size, cache_length, tree_draft_ids=None):
        """cache_length int32[1] on the device = P.  Returns (ids [T] -- entry 0 untouched --, positions [T],
        mask [T, W] as int64 bit patterns, parent [T])."""
        T = int(tree_size)
        dev = self.state.device
        W = mask_words(T)
        if tree_draft_ids is None:
            tree_draft_ids = torch.full((T,), -1, dtype=torch.int32, device=dev)
        pos = torch.empty(T, dtype=torch.int32, device=dev)
        mask = torch.empty((T, W), dtype=torch.int64, device=dev)
        parent = torch.empty(T, dtype=torch.int32, device=dev)
        _lib().draft_tree_finish(_ptr(self.state), self.k, self.num_iter, T, _ptr(cache_length), _ptr(self.remap),
                                 _ptr(tree_draft_ids), _ptr(pos), _ptr(mask), _ptr(parent), _stream())
        return tree_draft_ids, pos, mask, parent


def attention_plan(T, Hq, Hkv, max_kv_len, rope=False, block_window_size=0, num_splits=0):
    """(kernel names, KV splits, KV groups per workgroup, workgroups) of a tree-attention call of this shape."""
    buf = ctypes.create_string_buffer(160)
    ns, g, wg = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    _lib().tree_attention_plan(T, Hq, Hkv, int(max_kv_len), 1 if rope else 0, int(block_window_size), int(num_splits), buf, 160,
                               ctypes.byref(ns), ctypes.byref(g), ctypes.byref(wg))
    return buf.value.decode(), ns.value, g.value, wg.value


def head_plan(n, w):
    """(GEMM kernel name, workgroups) of a head call with n hidden rows on weight matrix w."""
    _, layout, V = _weight(w)
    H = w.H if isinstance(w, TiledWeight) else w.shape[1]
    buf = ctypes.create_string_buffer(96)
    wg = ctypes.c_int(0)
    _lib().head_plan(n, V, H, layout, buf, 96, ctypes.byref(wg))
    return buf.value.decode(), wg.value

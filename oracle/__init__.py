"""ctypes binding of the CPU oracle (``oracle/libcpmcu_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the
CPU-baseline leg of ``bench.py``; never by the product package.  All arrays are
numpy; fp16 tensors are ``np.float16`` (viewed as uint16 at the C boundary).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcpmcu_oracle.so")


def build(force=False):
    """Compile the oracle with g++ (no GPU dependencies)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B"] if force else ["make", "-C", _HERE])
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    c_p = ctypes.c_void_p
    i32, i64, f32 = ctypes.c_int, ctypes.c_int64, ctypes.c_float
    sigs = {
        "orc_f16_to_f32": (None, [c_p, c_p, i64]),
        "orc_f32_to_f16": (None, [c_p, c_p, i64]),
        "orc_f16_to_f32_sw": (None, [c_p, c_p, i64]),
        "orc_f32_to_f16_sw": (None, [c_p, c_p, i64]),
        "orc_num_threads": (i32, []),
        "orc_set_num_threads": (None, [i32]),
        "orc_tree_attention": (None, [c_p, c_p, c_p, c_p, i32, i32, i32, i32, i32, i32, i32, f32, c_p, c_p]),
        "orc_tree_attention_window": (None, [c_p, c_p, c_p, c_p, i32, i32, i32, i32, i32, i32, i32, i32, f32, c_p, c_p]),
        "orc_gather_rows": (None, [c_p, c_p, i32, i32, c_p]),
        "orc_lm_head": (None, [c_p, c_p, i32, i32, i32, i32, f32, c_p]),
        "orc_log_softmax": (None, [c_p, i32, i32, c_p, c_p]),
        "orc_log_softmax_apply": (None, [c_p, i32, i32, c_p, c_p]),
        "orc_topk": (None, [c_p, i32, i32, i32, c_p, c_p]),
        "orc_remap": (None, [c_p, i32, c_p, c_p]),
        "orc_argmax": (None, [c_p, i32, i32, c_p]),
        "orc_set_dtype": (None, [i32]),
        "orc_get_dtype": (i32, []),
        "orc_bf16_to_f32": (None, [c_p, c_p, i64]),
        "orc_f32_to_bf16": (None, [c_p, c_p, i64]),
        "orc_tree_accept": (i32, [i32, i32, c_p, c_p, c_p, i32, c_p, c_p, c_p, c_p]),
        "orc_kv_compact": (None, [c_p, i32, i32, i32, i32, c_p, c_p, c_p]),
        "orc_rope": (None, [i32, i32, i32, i32, c_p, c_p, c_p, c_p, c_p]),
        "orc_accept_commit": (None, [c_p, i32, i32, i32, i32, c_p, c_p, c_p, i32, c_p, c_p, c_p, c_p, c_p]),
        "orc_draft_tree_begin": (None, [i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p]),
        "orc_draft_tree_extend": (None, [i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p]),
        "orc_draft_tree_finish": (None, [i32, i32, i32, i32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = _load()


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def num_threads():
    return int(_lib.orc_num_threads())


def set_num_threads(n):
    _lib.orc_set_num_threads(int(n))


def f16_to_f32(x, software=False):
    x = _c(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    (_lib.orc_f16_to_f32_sw if software else _lib.orc_f16_to_f32)(_p(x), _p(out), x.size)
    return out


def f32_to_f16(x, software=False):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    (_lib.orc_f32_to_f16_sw if software else _lib.orc_f32_to_f16)(_p(x), _p(out), x.size)
    return out


def set_dtype(dtype):
    """Element type of every 16-bit tensor of the calls that follow: 0 / "f16" = IEEE binary16 (the default), 1 / "bf16" =
    bfloat16.  In bfloat16 mode the arrays still cross this module as numpy float16 arrays -- numpy has no bfloat16 --
    whose 16 bits are bfloat16 patterns: `encode` / `decode` convert between such containers and float32 values."""
    _lib.orc_set_dtype(1 if dtype in (1, "bf16") else 0)


def get_dtype():
    return int(_lib.orc_get_dtype())


def bf16_to_f32(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    _lib.orc_bf16_to_f32(_p(bits), _p(out), bits.size)
    return out


def f32_to_bf16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    _lib.orc_f32_to_bf16(_p(x), _p(out), x.size)
    return out


def decode(x):
    """float32 values of a 16-bit container (a numpy float16 array) under the element type in force."""
    x = np.ascontiguousarray(x)
    assert x.dtype == np.float16
    return bf16_to_f32(x.view(np.uint16)) if get_dtype() == 1 else x.astype(np.float32)


def encode(x):
    """The 16-bit container (numpy float16 array) of float32 values under the element type in force, rounded to nearest even."""
    x = np.ascontiguousarray(x, np.float32)
    return f32_to_bf16(x).view(np.float16) if get_dtype() == 1 else x.astype(np.float16)


def mask_words(T):
    return (T + 63) // 64


def tree_attention(q, k, v, mask, P, scale=None, return_lse=False, mask_k_range=None, block_window_size=0):
    """q [T,Hq,D] f16; k,v [P+T,Hkv,D] f16; mask [T,W] uint64 -> out [T,Hq,D] f16.
    mask_k_range (default T): number of trailing key columns the mask bits refer to.
    block_window_size (default 0 = none): the drafter layer's block sliding window, in tokens."""
    q = _c(q, np.float16)
    k = _c(k, np.float16)
    v = _c(v, np.float16)
    T, Hq, D = q.shape
    S, Hkv, _ = k.shape
    assert S == P + T and v.shape == k.shape
    mask = _c(mask, np.uint64).reshape(T, -1)
    W = mask.shape[1]
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    out = np.empty((T, Hq, D), np.float16)
    lse = np.empty((T, Hq), np.float32)
    R = T if mask_k_range is None else int(mask_k_range)
    assert T <= R <= S and W == (R + 63) // 64 or (W == 1 and R <= 64)
    _lib.orc_tree_attention_window(_p(q), _p(k), _p(v), _p(mask), T, P, Hq, Hkv, D, W, R, int(block_window_size),
                                   ctypes.c_float(scale), _p(out), _p(lse))
    return (out, lse) if return_lse else out


def gather_rows(src, remap):
    src = _c(src, np.float16)
    remap = _c(remap, np.int32)
    dst = np.empty((remap.size, src.shape[1]), np.float16)
    _lib.orc_gather_rows(_p(src), _p(remap), remap.size, src.shape[1], _p(dst))
    return dst


def lm_head(hid, w, head_scale=None):
    hid = _c(hid, np.float16)
    w = _c(w, np.float16)
    n, H = hid.shape
    V = w.shape[0]
    out = np.empty((n, V), np.float16)
    _lib.orc_lm_head(_p(hid), _p(w), n, V, H, 0 if head_scale is None else 1,
                     ctypes.c_float(1.0 if head_scale is None else head_scale), _p(out))
    return out


def log_softmax(x):
    """Returns (log-probs f16, m f32[n], lse f32[n]); the input is not modified."""
    x = np.array(x, dtype=np.float16, order="C", copy=True)
    n, dim = x.shape
    m = np.empty(n, np.float32)
    lse = np.empty(n, np.float32)
    _lib.orc_log_softmax(_p(x), n, dim, _p(m), _p(lse))
    return x, m, lse


def log_softmax_apply(x, m, lse):
    x = np.array(x, dtype=np.float16, order="C", copy=True)
    n, dim = x.shape
    m = _c(m, np.float32)
    lse = _c(lse, np.float32)
    _lib.orc_log_softmax_apply(_p(x), n, dim, _p(m), _p(lse))
    return x


def topk(x, top):
    x = _c(x, np.float16)
    n, dim = x.shape
    val = np.empty((n, top), np.float16)
    pos = np.empty((n, top), np.int32)
    _lib.orc_topk(_p(x), n, dim, top, _p(val), _p(pos))
    return val, pos


def remap(pos, table):
    pos = _c(pos, np.int32)
    table = _c(table, np.int32)
    out = np.empty(pos.shape, np.int32)
    _lib.orc_remap(_p(pos), pos.size, _p(table), _p(out))
    return out


def argmax(logits):
    logits = _c(logits, np.float16)
    n, V = logits.shape
    gt = np.empty(n, np.int32)
    _lib.orc_argmax(_p(logits), n, V, _p(gt))
    return gt


def tree_accept(pred, gt, pos, P, mask, parent):
    """Returns (a, best_node, path[:a])."""
    pred = _c(pred, np.int32)
    gt = _c(gt, np.int32)
    pos = _c(pos, np.int32)
    parent = _c(parent, np.int32)
    T = pred.size
    mask = _c(mask, np.uint64).reshape(T, -1)
    W = mask.shape[1]
    best = np.zeros(2, np.int32)
    path = np.full(T, -1, np.int32)
    a = _lib.orc_tree_accept(T, W, _p(pred), _p(gt), _p(pos), int(P), _p(mask), _p(parent), _p(best), _p(path))
    return int(a), int(best[1]), path[:a].copy()


def kv_compact(caches, P, path, gt):
    """caches: list of [rows,row_halves] f16 arrays, modified in place. Returns accepted ids."""
    path = _c(path, np.int32)
    gt = _c(gt, np.int32)
    a = path.size
    for c in caches:
        assert c.dtype == np.float16 and c.flags.c_contiguous
    row_halves = caches[0].shape[1]
    ptrs = (ctypes.c_void_p * len(caches))(*[c.ctypes.data for c in caches])
    ids = np.empty(a, np.int32)
    _lib.orc_kv_compact(ptrs, len(caches), row_halves, int(P), a, _p(path), _p(gt), _p(ids))
    return ids


def rope(q, k, pos=None, inv_freq=None, table=None):
    """Rotary embedding (src/model/rotary.cuh:7-34) of q [T,Hq,D] and k [T,Hkv,D]; returns rotated copies.
    Angles from (pos, inv_freq), or from a given table [T, D/2, 2] of (cos, sin)."""
    q = np.array(q, dtype=np.float16, order="C", copy=True)
    k = np.array(k, dtype=np.float16, order="C", copy=True)
    T, Hq, Dh = q.shape
    half = Dh // 2
    if table is not None:
        table = _c(table, np.float32).reshape(T, half, 2)
    else:
        pos = _c(pos, np.int32)
        inv_freq = _c(inv_freq, np.float32)
        assert inv_freq.size == half
    _lib.orc_rope(T, Hq, k.shape[1], half, _p(inv_freq), _p(pos), _p(table), _p(q), _p(k))
    return q, k


def accept_commit(caches, P, path, gt, hidden=None):
    """verify() after the acceptance (src/model/minicpm4/minicpm4_eagle.cuh:403-411) on host arrays; caches are
    modified in place.  Returns dict(prev_hidden [a,H] or None, next_pos [a], result [1+a] = (a, ids), new_length, next_root)."""
    path = _c(path, np.int32)
    gt = _c(gt, np.int32)
    a = path.size
    for c in caches:
        assert c.dtype == np.float16 and c.flags.c_contiguous
    row_halves = caches[0].shape[1]
    ptrs = (ctypes.c_void_p * len(caches))(*[c.ctypes.data for c in caches])
    H = 0
    prev = None
    if hidden is not None:
        hidden = _c(hidden, np.float16)
        H = hidden.shape[1]
        prev = np.zeros((a, H), np.float16)
    next_pos = np.empty(a, np.int32)
    result = np.empty(1 + a, np.int32)
    new_len = np.zeros(1, np.int32)
    root = np.zeros(1, np.int32)
    _lib.orc_accept_commit(ptrs, len(caches), row_halves, int(P), a, _p(path), _p(gt), _p(hidden), H, _p(prev),
                           _p(next_pos), _p(result), _p(new_len), _p(root))
    return dict(prev_hidden=prev, next_pos=next_pos, result=result, new_length=int(new_len[0]), next_root=int(root[0]))


class DraftTree:
    """Tree bookkeeping of the drafter (src/model/minicpm4/minicpm4_eagle.cuh:319-393) on host arrays."""

    def __init__(self, k, num_iter, token_id_remap=None):
        self.k, self.num_iter = int(k), int(num_iter)
        total = k + (num_iter - 1) * k * k
        self.remap = None if token_id_remap is None else _c(token_id_remap, np.int32)
        self.tried_val = np.zeros(total, np.float16)
        self.tried_pos = np.zeros(total, np.int32)
        self.tried_parent = np.zeros(max(1, k * (num_iter - 1)), np.int32)
        self.cum = np.zeros(k, np.float16)
        self.mask = np.zeros(k, np.uint64)

    def begin(self, val, pos):
        """val, pos [k] -> next_ids [k]."""
        val, pos = _c(val, np.float16), _c(pos, np.int32)
        ids = np.empty(self.k, np.int32)
        _lib.orc_draft_tree_begin(self.k, _p(val), _p(pos), _p(self.remap), _p(self.tried_val), _p(self.tried_pos),
                                  _p(self.cum), _p(self.mask), _p(ids))
        return ids

    def extend(self, d, val, pos):
        """val, pos [k, k] of iteration d >= 1 -> (next_ids [k], parent_rows [k], cumulated val [k, k])."""
        val = np.array(val, dtype=np.float16, order="C", copy=True)
        pos = _c(pos, np.int32)
        ids = np.empty(self.k, np.int32)
        rows = np.empty(self.k, np.int32)
        _lib.orc_draft_tree_extend(self.k, int(d), _p(val), _p(pos), _p(self.remap), _p(self.tried_val), _p(self.tried_pos),
                                   _p(self.tried_parent), _p(self.cum), _p(self.mask), _p(ids), _p(rows))
        return ids, rows, val

    def finish(self, T, P):
        """-> (ids [T] with ids[0] = -1, positions [T], mask [T, W], parent [T])."""
        W = (T + 63) // 64
        ids = np.full(T, -1, np.int32)
        tpos = np.empty(T, np.int32)
        tmask = np.zeros((T, W), np.uint64)
        tpar = np.empty(T, np.int32)
        _lib.orc_draft_tree_finish(self.k, self.num_iter, int(T), int(P), _p(self.remap), _p(self.tried_val), _p(self.tried_pos),
                                   _p(self.tried_parent), _p(ids), _p(tpos), _p(tmask), _p(tpar))
        return ids, tpos, tmask, tpar

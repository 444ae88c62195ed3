"""Paged KV cache of the verify path: pools, page table and the token <-> slot arithmetic.

Layout (chosen for the gfx950 kernels; the reference keeps flat per-layer buffers,
src/model/kvcache.cuh:18-25, and its layout never crosses the boundary):

* page = 256 tokens; ``block_table[i]`` = physical page of logical page ``i``; one table for all
  layers, one K pool and one V pool per layer
* K pool ``[pages, Hkv, 256, 128]`` fp16 -- row-major token rows
* V pool ``[pages, Hkv, 128, 256]`` fp16 -- transposed; inside each aligned group of 16 tokens the
  slot of token ``t`` is ``t`` with bits 2 and 3 swapped (``v_slot``)

The ``*_logical`` helpers move whole token rows with plain torch indexing; they are the independent
check of the HIP append / compaction kernels and the way tests look at a cache.
"""
import torch

PAGE = 256
HEAD_DIM = 128


def v_slot(t):
    """Slot of token index ``t`` inside a transposed V page (works on ints and integer tensors)."""
    return (t & ~12) | ((t & 4) << 1) | ((t & 8) >> 1)


class PagedKVCache:
    def __init__(self, num_layers, num_kv_heads, num_pages, device="cuda", block_table=None, fill=None):
        self.num_layers = num_layers
        self.Hkv = num_kv_heads
        self.num_pages = num_pages
        self.device = torch.device(device)
        mk = torch.zeros if fill is None else (lambda *s, **k: torch.full(s, fill, **k))
        self.k = [mk(num_pages, num_kv_heads, PAGE, HEAD_DIM, dtype=torch.float16, device=self.device) for _ in range(num_layers)]
        self.v = [mk(num_pages, num_kv_heads, HEAD_DIM, PAGE, dtype=torch.float16, device=self.device) for _ in range(num_layers)]
        if block_table is None:
            block_table = torch.arange(num_pages, dtype=torch.int32)
        self.block_table = torch.as_tensor(block_table, dtype=torch.int32).to(self.device).contiguous()
        assert self.block_table.numel() <= num_pages
        # device arrays of pool pointers, as the compaction kernel takes them
        self.k_ptrs = torch.tensor([t.data_ptr() for t in self.k], dtype=torch.int64, device=self.device)
        self.v_ptrs = torch.tensor([t.data_ptr() for t in self.v], dtype=torch.int64, device=self.device)

    @classmethod
    def from_pools(cls, k_pools, v_pools, block_table):
        """A cache over pools that already exist (tensor views [pages, Hkv, 256, 128] / [pages, Hkv, 128, 256])."""
        self = cls.__new__(cls)
        self.num_layers = len(k_pools)
        self.Hkv = k_pools[0].shape[1]
        self.num_pages = k_pools[0].shape[0]
        self.device = k_pools[0].device
        self.k, self.v = list(k_pools), list(v_pools)
        self.block_table = block_table
        self.k_ptrs = torch.tensor([t.data_ptr() for t in self.k], dtype=torch.int64, device=self.device)
        self.v_ptrs = torch.tensor([t.data_ptr() for t in self.v], dtype=torch.int64, device=self.device)
        return self

    @property
    def capacity(self):
        return self.block_table.numel() * PAGE

    def _locate(self, start, n):
        tok = torch.arange(start, start + n, device=self.device)
        page = self.block_table[tok // PAGE].long()
        slot = tok % PAGE
        return page, slot

    def write_logical(self, layer, start, k_rows, v_rows):
        """k_rows, v_rows: [n, Hkv, 128] -> token positions [start, start + n)."""
        n = k_rows.shape[0]
        page, slot = self._locate(start, n)
        self.k[layer][page, :, slot, :] = k_rows.to(self.device, torch.float16).reshape(n, self.Hkv, HEAD_DIM)
        self.v[layer][page, :, :, v_slot(slot)] = v_rows.to(self.device, torch.float16).reshape(n, self.Hkv, HEAD_DIM)

    def read_logical(self, layer, start, n):
        """-> (k [n, Hkv, 128], v [n, Hkv, 128]) of token positions [start, start + n)."""
        page, slot = self._locate(start, n)
        return self.k[layer][page, :, slot, :].clone(), self.v[layer][page, :, :, v_slot(slot)].clone()

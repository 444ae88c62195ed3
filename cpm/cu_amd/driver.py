"""Host-side counterpart of the reference's speculative step for the verify path.

One verify step, as the reference drives it (cpmcu/speculative/tree_drafter.py:222-250 around
cpmcu/llm.py:263-283), restricted to the operators that are on the path:

    for every layer:  append the T tree rows' K/V at cache rows [P, P+T)   (src/model/attn.cuh:200)   } one fused
                      tree attention of the T queries over P + T keys      (src/model/attn.cuh:204-229) } kernel
    target head on the T hidden rows + arg-max  -> gt                      (src/model/model.cuh:164, tree_drafter.py:233)
    greedy acceptance -> (a, path)                                         (src/model/tree_drafter.cuh:5-46)
    compaction of the accepted rows in every layer, pred[:a] <- ids        (src/model/tree_drafter.cuh:48-77)

The dense projections / FFN between those calls are not part of the path, so the per-layer Q, new
K/V rows and the final hidden rows are inputs.  Everything is enqueued on torch's current stream
with no host synchronisation, so a whole step can be captured into one HIP graph and replayed.

With ``commit=True`` the tail of the step is the one-call form of verify() (``ops.accept_commit``):
the prefix length and the attention's total length advance on the device, the accepted hidden rows
are gathered for the drafter, and (accept length, ids) land in pinned host memory -- so consecutive
steps need no host write at all and ``GraphedSteps`` replays one captured graph per padded length,
the reference's ``(padded_length, T)`` graph key (src/entry.cu:475-492).
"""
import torch

from . import ops


class VerifyStep:
    """fused=True (default): the head leaves its arg-max as per-workgroup partials and ONE launch finishes it,
    accepts, compacts every cache and writes the ids (``ops.verify_tail``); the draft ids are read where the
    caller keeps them.  fused=False keeps the operator-by-operator tail (arg-max finish, ``tree_accept``,
    ``kv_compact`` / ``accept_commit``), which needs the draft ids copied into ``pred`` first."""

    def __init__(self, cache, lm_head, tree_mask, tree_parent, tree_positions, prefix_len, head_scale=None, commit=False, fused=True):
        dev = cache.device
        self.cache = cache
        self.w = lm_head
        self.T = tree_parent.numel()
        self.mask = tree_mask
        self.parent = tree_parent
        self.pos = tree_positions
        self.head_scale = head_scale
        self.P = int(prefix_len)
        self.cache_length = torch.tensor([self.P], dtype=torch.int32, device=dev)         # P
        self.kv_len = torch.tensor([self.P + self.T], dtype=torch.int32, device=dev)       # P + T (cpmcu/llm.py:272)
        self.max_kv_len = (self.P + self.T + 127) // 128 * 128                            # padded_length (cpmcu/llm.py:273)
        self.gt = torch.empty(self.T, dtype=torch.int32, device=dev)
        self.best = torch.zeros(2, dtype=torch.int32, device=dev)
        self.pred = torch.empty(self.T, dtype=torch.int32, device=dev)
        self.attn_out = None
        self.commit = bool(commit)
        self.fused = bool(fused)
        # only the fused tail advances the tree positions with the lengths; the operator-by-operator tail would leave
        # them behind the device-side prefix length from the second step on
        assert self.fused or not self.commit, "commit=True needs the fused tail"
        self.path = torch.zeros(self.T, dtype=torch.int32, device=dev)
        if self.commit:
            self.prev_hidden = None  # allocated at the first step, when the hidden size is known
            self.next_positions = torch.zeros(self.T, dtype=torch.int32, device=dev)
            self.packed = torch.zeros(1 + self.T, dtype=torch.int32).pin_memory()  # (a, ids): written by the GPU

    def enqueue(self, q_layers, k_new_layers, v_new_layers, hidden, draft_ids, attn_out=None, splits=0):
        """Enqueue one full verify step.  q_layers[l] [T,Hq,128]; k/v_new_layers[l] [T,Hkv,128];
        hidden [T,H]; draft_ids int32[T].  Results: self.best (a, node), self.pred[:a] accepted ids."""
        c = self.cache
        for l in range(c.num_layers):
            out = None if attn_out is None else attn_out[l]
            # the KV append of the T tree rows is fused into the attention kernel
            o = ops.tree_attention(q_layers[l], c, l, self.kv_len, self.max_kv_len, self.mask, num_splits=splits, out=out,
                                   k_new=k_new_layers[l], v_new=v_new_layers[l])
            if attn_out is None:
                self.attn_out = o
        if self.fused:
            parts = ops.lm_head_partials(hidden, self.w, head_scale=self.head_scale)
            if self.commit and self.prev_hidden is None:
                self.prev_hidden = torch.zeros((self.T, hidden.shape[1]), dtype=torch.float16, device=hidden.device)
            ops.verify_tail(c, draft_ids, parts, self.pos, self.cache_length, self.mask, self.parent,
                            hidden=hidden if self.commit else None, prev_hidden=self.prev_hidden if self.commit else None,
                            gt_out=self.gt, best=self.best, path=self.path, accepted_ids=self.pred,
                            next_position_ids=self.next_positions if self.commit else None,
                            result=self.packed if self.commit else None)
            if self.commit:
                # lengths and tree positions advance on the device: the next step of the same tree shape needs no host write
                ops.verify_tail_inplace(self.best, self.pred, cache_length=self.cache_length, kv_len=self.kv_len,
                                        position_ids=self.pos, advance_length=True)
            return
        ops.lm_head_argmax(hidden, self.w, head_scale=self.head_scale, gt=self.gt)
        self.pred.copy_(draft_ids)
        ops.tree_accept(self.pred, self.gt, self.pos, self.cache_length, self.mask, self.parent, best=self.best)
        if not self.commit:
            ops.kv_compact(c, self.pred, self.gt, self.cache_length, self.best, self.T)
            return
        if self.prev_hidden is None:
            self.prev_hidden = torch.zeros((self.T, hidden.shape[1]), dtype=torch.float16, device=hidden.device)
        ops.accept_commit(c, self.pred, self.gt, self.cache_length, self.best, self.T, hidden=hidden,
                          prev_hidden=self.prev_hidden, next_position_ids=self.next_positions, result=self.packed,
                          advance_length=True, kv_len=self.kv_len)

    def result(self):
        """(accept length, accepted token ids) after one synchronisation.  With commit the GPU has
        already written both into pinned host memory; otherwise they are read back from the device."""
        torch.cuda.current_stream().synchronize()
        if self.commit:
            a = int(self.packed[0])
            return a, self.packed[1:1 + a].numpy().copy()
        a = int(self.best[0].item())
        return a, self.pred[:a].cpu().numpy()


class GraphedSteps:
    """Consecutive verify steps as replays of captured HIP graphs, one graph per padded length
    (the reference captures its decode graph per (padded_length, T), src/entry.cu:475-492).

    The step's inputs live in static device buffers that the caller refills before each replay
    (``buffers()``); lengths advance on the device (VerifyStep with commit), so the host only has to
    keep an upper bound of the prefix length to know when a longer padded length is due -- it learns
    the exact value from every step's result anyway.
    """

    def __init__(self, step, num_layers, Hq, Hkv, hidden_size, pad_to=1024):
        assert step.commit, "graph replay needs the device-side length advance of commit=True"
        dev = step.cache.device
        T = step.T
        f16 = dict(dtype=torch.float16, device=dev)
        self.step = step
        self.pad_to = int(pad_to)
        self.q = [torch.zeros((T, Hq, 128), **f16) for _ in range(num_layers)]
        self.k_new = [torch.zeros((T, Hkv, 128), **f16) for _ in range(num_layers)]
        self.v_new = [torch.zeros((T, Hkv, 128), **f16) for _ in range(num_layers)]
        self.attn_out = [torch.zeros((T, Hq, 128), **f16) for _ in range(num_layers)]
        self.hidden = torch.zeros((T, hidden_size), **f16)
        self.draft_ids = torch.zeros(T, dtype=torch.int32, device=dev)
        step.prev_hidden = torch.zeros((T, hidden_size), **f16)
        self.graphs = {}
        self.stream = torch.cuda.Stream()
        self.prefix_bound = step.P  # host-side upper bound of the device's prefix length

    def buffers(self):
        return self.q, self.k_new, self.v_new, self.hidden, self.draft_ids

    def _padded(self):
        need = self.prefix_bound + self.step.T
        return (need + self.pad_to - 1) // self.pad_to * self.pad_to

    def run(self):
        """Replay (capturing first, if this padded length is new) one step; returns (a, ids)."""
        st = self.step
        padded = self._padded()
        assert padded <= st.cache.num_pages * 256, "the paged cache is too small for this padded length"
        if padded not in self.graphs:
            # capture enqueues without running: the device scalars keep their values
            st.max_kv_len = padded
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(self.stream):
                with torch.cuda.graph(g, stream=self.stream):
                    st.enqueue(self.q, self.k_new, self.v_new, self.hidden, self.draft_ids, attn_out=self.attn_out)
            self.graphs[padded] = g
        with torch.cuda.stream(self.stream):
            self.graphs[padded].replay()
        self.stream.synchronize()
        a = int(st.packed[0])
        self.prefix_bound += a
        return a, st.packed[1:1 + a].numpy().copy()

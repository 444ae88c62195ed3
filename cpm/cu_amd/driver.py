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
"""
import torch

from . import ops


class VerifyStep:
    def __init__(self, cache, lm_head, tree_mask, tree_parent, tree_positions, prefix_len, head_scale=None):
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
        ops.lm_head_argmax(hidden, self.w, head_scale=self.head_scale, gt=self.gt)
        self.pred.copy_(draft_ids)
        ops.tree_accept(self.pred, self.gt, self.pos, self.cache_length, self.mask, self.parent, best=self.best)
        ops.kv_compact(c, self.pred, self.gt, self.cache_length, self.best, self.T)

    def result(self):
        """Single D2H read of the step: (accept length, accepted token ids)."""
        torch.cuda.current_stream().synchronize()
        a = int(self.best[0].item())
        return a, self.pred[:a].cpu().numpy()

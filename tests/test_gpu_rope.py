"""Rotary embedding of the tree rows (src/model/rotary.cuh:7-34): the per-step (cos, sin) table, the in-place
operator, and the form fused into tree attention (queries rotated in registers, appended K rows rotated
on their way into the cache), all through the C-ABI.

The rotation itself is compared bit for bit with the oracle run on the device's own table (staged);
the table is compared with float32 cos/sin of the same float32 angle; and the fused attention is
compared with "rotate in place, then attend" on the device and with the oracle end to end.
"""
import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 2, 128
HALF = D // 2


def _inv_freq(base=10000.0):
    return (base ** (-np.arange(HALF, dtype=np.float64) / HALF)).astype(np.float32)


def test_rope_table_and_in_place_operator(gpu, orc):
    from cpm.cu_amd import ops
    torch = gpu
    T = 60
    pos = np.concatenate([[0, 1, 5], synth.rng(1, 1).integers(0, 131072, T - 3)]).astype(np.int32)
    inv_freq = _inv_freq()
    table = ops.rope_table(to_dev(torch, pos), to_dev(torch, inv_freq))
    torch.cuda.synchronize()
    tab = to_np(table)
    ang = (pos.astype(np.float32)[:, None] * inv_freq[None, :]).astype(np.float32)  # the float32 product the kernel forms
    assert np.max(np.abs(tab[..., 0] - np.cos(ang.astype(np.float64)))) <= 2e-7 + 1e-6
    assert np.max(np.abs(tab[..., 1] - np.sin(ang.astype(np.float64)))) <= 2e-7 + 1e-6
    assert np.array_equal(tab[0, :, 0], np.ones(HALF, np.float32)) and np.array_equal(tab[0, :, 1], np.zeros(HALF, np.float32))

    q = synth.normal_f16((T, HQ, D), 3, 1)
    k = synth.normal_f16((T, HKV, D), 3, 2)
    dq, dk = to_dev(torch, q), to_dev(torch, k)
    ops.rope_apply_(table, dq, dk)
    torch.cuda.synchronize()
    q_st, k_st = orc.rope(q, k, table=tab)  # staged: same table, same arithmetic -> same bits
    assert np.array_equal(to_np(dq).view(np.uint16), q_st.view(np.uint16))
    assert np.array_equal(to_np(dk).view(np.uint16), k_st.view(np.uint16))
    q_or, k_or = orc.rope(q, k, pos, inv_freq)  # end to end: host cosf/sinf may differ in the last float32 bit
    assert_close_f16(to_np(dq), q_or, "rotated q")
    assert_close_f16(to_np(dk), k_or, "rotated k")


@pytest.mark.parametrize("P,T,groups", [(1000, 60, "2"), (4096 - 30, 60, "2"), (300, 17, "1"), (70000, 64, "1"), (0, 9, "2")])
def test_attention_with_fused_rope(gpu, orc, set_option, P, T, groups):
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    set_option("attn_kv_groups", int(groups))
    seed = P + T
    tree = synth.random_tree(T, seed, max_children=4, max_depth=8)
    mask = to_dev(torch, tree.mask)
    S = P + T
    npages = (S + 255) // 256 + 1
    table_np = synth.rng(seed, 4).permutation(npages).astype(np.int32)
    kp = synth.normal_f16((P, HKV, D), seed, 10)
    vp = synth.normal_f16((P, HKV, D), seed, 11)
    q = synth.normal_f16((T, HQ, D), seed, 1)
    kn = synth.normal_f16((T, HKV, D), seed, 2)
    vn = synth.normal_f16((T, HKV, D), seed, 3)
    pos = tree.positions(P)
    inv_freq = _inv_freq()
    rope = ops.rope_table(to_dev(torch, pos), to_dev(torch, inv_freq))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    max_len = (S + 127) // 128 * 128

    def fresh():
        c = PagedKVCache(1, HKV, npages, block_table=table_np)
        if P:
            c.write_logical(0, 0, to_dev(torch, kp), to_dev(torch, vp))
        return c

    # fused: unrotated q / k_new in, rotation inside the kernel
    c1 = fresh()
    dq, dkn, dvn = to_dev(torch, q), to_dev(torch, kn), to_dev(torch, vn)
    out1 = ops.tree_attention(dq, c1, 0, kv_len, max_len, mask, k_new=dkn, v_new=dvn, rope=rope)
    # reference order on the device: rotate in place, then the plain fused-append attention
    c2 = fresh()
    dq2, dkn2 = to_dev(torch, q), to_dev(torch, kn)
    ops.rope_apply_(rope, dq2, dkn2)
    out2 = ops.tree_attention(dq2, c2, 0, kv_len, max_len, mask, k_new=dkn2, v_new=dvn)
    torch.cuda.synchronize()
    assert np.array_equal(to_np(dq).view(np.uint16), q.view(np.uint16)), "the fused form must not modify q"
    assert np.array_equal(to_np(dkn).view(np.uint16), kn.view(np.uint16)), "the fused form must not modify k_new"
    # same rotated operands and identical cache contents; the outputs agree to fp16 rounding only, because
    # the fused form gives the split that also rotates K a smaller share of the tiles (other split boundaries)
    assert_close_f16(to_np(out1), to_np(out2), "fused rope vs rotate-then-attend", atol=4e-3, rtol=4e-3)
    k1, v1 = c1.read_logical(0, 0, S)
    k2, v2 = c2.read_logical(0, 0, S)
    assert np.array_equal(to_np(k1).view(np.uint16), to_np(k2).view(np.uint16))
    assert np.array_equal(to_np(v1).view(np.uint16), to_np(v2).view(np.uint16))
    # the appended K rows are the oracle's rotation of k_new with the device's table, bit for bit
    _, k_st = orc.rope(q, kn, table=to_np(rope))
    assert np.array_equal(to_np(k1)[P:].view(np.uint16), k_st.view(np.uint16))
    # end to end against the oracle
    q_or, k_or = orc.rope(q, kn, pos, inv_freq)
    k_all = np.concatenate([kp, k_or], 0) if P else k_or
    v_all = np.concatenate([vp, vn], 0) if P else vn
    ref = orc.tree_attention(q_or, k_all, v_all, tree.mask, P)
    assert_close_f16(to_np(out1), ref, "attention with fused rope")


def test_fused_rope_without_append_rotates_q_only(gpu, orc):
    """k_new = None: the keys are already in the cache (rotated when they were appended); only q rotates."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    P, T, seed = 500, 12, 9
    S = P + T
    tree = synth.chain_tree(T)
    k = synth.normal_f16((S, HKV, D), seed, 10)
    v = synth.normal_f16((S, HKV, D), seed, 11)
    q = synth.normal_f16((T, HQ, D), seed, 1)
    cache = PagedKVCache(1, HKV, (S + 255) // 256 + 1)
    cache.write_logical(0, 0, to_dev(torch, k), to_dev(torch, v))
    pos = tree.positions(P)
    inv_freq = _inv_freq()
    rope = ops.rope_table(to_dev(torch, pos), to_dev(torch, inv_freq))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, to_dev(torch, tree.mask), rope=rope)
    torch.cuda.synchronize()
    q_st, _ = orc.rope(q, k[:T], table=to_np(rope))
    ref = orc.tree_attention(q_st, k, v, tree.mask, P)
    assert_close_f16(to_np(out), ref, "attention with rotated q only")
    kc, _ = cache.read_logical(0, 0, S)
    assert np.array_equal(to_np(kc).view(np.uint16), k.view(np.uint16))

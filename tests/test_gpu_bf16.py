"""The path in bfloat16 (torch_dtype = 1 of src/entry.cu:26-59) against the CPU oracle in bfloat16.

numpy has no bfloat16: host arrays are float16-typed containers whose 16 bits are bfloat16 patterns (`orc.encode` /
`orc.decode` convert to and from float32), and the same containers travel to the device.  Integer results are bit-exact as
in fp16; floating-point results are compared within max-abs 2e-2 and a normalised-max error of 2e-2 -- one bfloat16 ulp
is 2^-8 of the value, eight times an fp16 ulp, and a result that lands on the other side of a rounding boundary (the
fp32 sums are taken in another order on the device) is off by a whole one.
"""
import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 2, 128
RTOL_BF16 = 2e-2


@pytest.fixture
def bf16(gpu, orc, set_option):
    """Library and oracle in bfloat16 for one test."""
    set_option("dtype", 1)
    orc.set_dtype("bf16")
    yield
    orc.set_dtype("f16")


def normal_bf16(orc, shape, seed, stream, std=1.0):
    return orc.encode(synth.rng(seed, stream).standard_normal(shape, dtype=np.float32) * std)


@pytest.mark.parametrize("groups", [2, 1])
@pytest.mark.parametrize("P,T,rope", [(1024, 16, False), (4096, 60, False), (4096 - 37, 60, True), (700, 128, False)])
def test_bf16_tree_attention_with_fused_append(gpu, orc, bf16, set_option, groups, P, T, rope):
    torch = gpu
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    set_option("attn_kv_groups", groups)
    tree = synth.eagle_tree(6, 10, T, seed=P) if T > 16 else synth.eagle_tree(4, 4, T, seed=P)
    S = P + T
    q = normal_bf16(orc, (T, HQ, D), P, 1)
    k = normal_bf16(orc, (S, HKV, D), P, 2)
    v = normal_bf16(orc, (S, HKV, D), P, 3)
    npages = (S + 255) // 256 + 1
    cache = PagedKVCache(1, HKV, npages, block_table=synth.rng(P, 4).permutation(npages).astype(np.int32))
    cache.write_logical(0, 0, to_dev(torch, k[:P]), to_dev(torch, v[:P]))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    table = None
    q_ref, k_ref = q, k
    if rope:
        pos = np.arange(P, P + T, dtype=np.int32)
        inv_freq = (1.0 / (10000.0 ** (np.arange(0, D, 2, dtype=np.float32) / D))).astype(np.float32)
        table = ops.rope_table(to_dev(torch, pos), to_dev(torch, inv_freq))
        q_ref, k_rot = orc.rope(q, k[P:], table=to_np(table))
        k_ref = np.concatenate([k[:P], k_rot])
    out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, to_dev(torch, tree.mask), k_new=to_dev(torch, k[P:]),
                             v_new=to_dev(torch, v[P:]), rope=table)
    torch.cuda.synchronize()
    ref = orc.tree_attention(q_ref, k_ref, v, tree.mask, P)
    assert_close_f16(orc.decode(to_np(out)), orc.decode(ref), "bf16 attention P=%d T=%d" % (P, T), rtol=RTOL_BF16)
    kc, vc = cache.read_logical(0, 0, S)
    assert np.array_equal(to_np(kc).view(np.uint16), k_ref.view(np.uint16))
    assert np.array_equal(to_np(vc).view(np.uint16), v.view(np.uint16))

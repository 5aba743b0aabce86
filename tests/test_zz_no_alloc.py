"""akv_paged_attn_static: the attention entry point that allocates nothing (its scratch is a fixed
array inside the library's device image) against akv_paged_attn on the same inputs, through the C
ABI: two calls in a row, the second with a smaller batch and shorter contexts, so that whatever the
first call left in the shared array must not reach the second call's result."""
import numpy as np
import pytest
import torch

import aitherkvcache_amd as akv
from aitherkvcache_amd import _lib
from oracle import tq_oracle as O
from tests.test_gpu_attention import build_cache, make_tq, oracle_out, t, within_tol

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits", [4, 3])
def test_static_scratch_entry_matches_workspace_entry(golden, dev, bits):
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(5000 + bits)
    NB, KVH, QH = 160, 8, 32
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, KVH, bits)
    attn = akv.TQPagedAttention(tq, num_query_heads=QH)
    assert _lib.lib().akv_paged_attn_static_scratch_bytes() == 32 << 20
    for S, max_ctx, width in ((12, 900, 60), (3, 70, 8)):
        ctx = rng.integers(1, max_ctx, size=S).astype(np.int64)
        ctx[0] = max_ctx
        tables = np.stack([rng.permutation(NB)[:width] for _ in range(S)]).astype(np.int64)
        q = t(rng.standard_normal((S, QH, 128)).astype(np.float16), dev)
        tb, cl = t(tables, dev), t(ctx, dev)
        want = attn.forward(q, kp, kn, vp, vn, tb, cl, block_size=16, num_kv_heads=KVH)
        out = torch.full_like(want, float("nan"))
        torch.cuda.synchronize()
        count = lambda: torch.cuda.memory_stats(dev)["allocation.all.allocated"]   # requests to torch's allocator
        before = count()
        got = attn.forward_no_alloc(q, kp, kn, vp, vn, tb, cl, out, block_size=16, num_kv_heads=KVH)
        torch.cuda.synchronize()
        assert count() == before
        assert got is out
        assert torch.equal(got, want), f"S={S}: max diff {(got.float() - want.float()).abs().max().item():.3e}"
        ref = oracle_out(q.cpu().numpy(), kp, kn, vp, vn, tables, ctx, golden, bits)
        assert within_tol(got.cpu().numpy(), ref)
        assert attn.last_call_status() == 0           # read from the built-in array's own status word
    with pytest.raises(ValueError, match="float32 norms"):
        attn.forward_no_alloc(q, kp, kn.half(), vp, vn, tb, cl, out, block_size=16, num_kv_heads=KVH)


def test_static_scratch_entry_rejects_oversized_batches(golden, dev):
    tq = make_tq(golden, dev, 4)
    attn = akv.TQPagedAttention(tq, num_query_heads=32)
    S = 400
    q = torch.zeros(S, 32, 128, dtype=torch.float16, device=dev)
    kp = torch.zeros(4, 16, 8, 64, dtype=torch.uint8, device=dev)
    kn = torch.zeros(4, 16, 8, device=dev)
    tb = torch.zeros(S, 2, dtype=torch.int32, device=dev)
    cl = torch.ones(S, dtype=torch.int32, device=dev)
    with pytest.raises(_lib.AkvError, match="scratch"):
        attn.forward_no_alloc(q, kp, kn, kp, kn, tb, cl, torch.empty_like(q), block_size=16, num_kv_heads=8)

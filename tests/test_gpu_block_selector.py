"""Block selector kernels (representatives, scores, top-k) against the reference's vectors and the oracle."""
import os

import numpy as np
import pytest
import torch

import aitherkvcache_amd as akv
from aitherkvcache_amd.block_selector import BlockRepresentativeCache, BlockSelector, score_blocks, select_blocks
from oracle import tq_oracle as O
from tests.util import kv_like

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def bsel():
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_block_selector.npz"))


def t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def test_representatives_golden(bsel, dev):
    cache = BlockRepresentativeCache(12, 2, 64, dev, t(bsel["centroids"], dev))
    for call in range(3):
        bi = bsel[f"rep_bi_{call}"]
        idx = t(bi, dev) if call != 1 else t(bi, dev).int()
        cache.update(idx, t(bsel[f"rep_pos_{call}"], dev), t(bsel[f"rep_kp_{call}"], dev), t(bsel[f"rep_kn_{call}"], dev))
        cache.finalize(t(np.unique(bi), dev))
        assert np.array_equal(cache._counts.cpu().numpy(), bsel[f"rep_counts_after_{call}"])
        # sums of up to ~10 terms of size ~10 in the order the atomics land: absolute slack for cancelling terms
        np.testing.assert_allclose(cache.rep_even.cpu().numpy(), bsel[f"rep_even_after_{call}"], rtol=3e-6, atol=5e-6)
        np.testing.assert_allclose(cache.rep_odd.cpu().numpy(), bsel[f"rep_odd_after_{call}"], rtol=3e-6, atol=5e-6)
    cache.clear_blocks(torch.tensor([3, 4], device=dev))
    cache.finalize()
    assert np.array_equal(cache._counts.cpu().numpy(), bsel["rep_counts_cleared"])
    np.testing.assert_allclose(cache.rep_even.cpu().numpy(), bsel["rep_even_cleared"], rtol=3e-6, atol=5e-6)
    # ids outside the cache are skipped, an empty update is a no-op
    before = cache._acc_even.clone()
    cache.update(torch.tensor([-1, 99], device=dev), torch.zeros(2, dtype=torch.long, device=dev),
                 torch.zeros(2, 2, 64, dtype=torch.uint8, device=dev), torch.ones(2, 2, device=dev))
    cache.update(torch.empty(0, dtype=torch.long, device=dev), torch.empty(0, dtype=torch.long, device=dev),
                 torch.empty(0, 2, 64, dtype=torch.uint8, device=dev), torch.empty(0, 2, device=dev))
    assert torch.equal(before, cache._acc_even)


@pytest.mark.parametrize("itype", [torch.int64, torch.int32])
def test_scores_and_selection_golden(bsel, dev, itype):
    bt, ctx = t(bsel["sel_bt"], dev).to(itype), t(bsel["sel_ctx"], dev).to(itype)
    sc = score_blocks(t(bsel["sel_q_even"], dev), t(bsel["sel_q_odd"], dev), t(bsel["sel_rep_even"], dev),
                      t(bsel["sel_rep_odd"], dev), bt, ctx, 4, 16)
    ref = bsel["sel_scores"]
    got = sc.cpu().numpy()
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert np.max(np.abs(got[fin] - ref[fin])) <= 3e-5
    nb = (bsel["sel_ctx"] + 15) // 16
    for tag, ms, sinks, recents in (("10", 10, 2, 2), ("40", 40, 2, 2), ("120", 120, 2, 2), ("12_s1r3", 12, 1, 3)):
        # the reference's scores go in, so that the selection is compared on identical keys
        fbt, fcl = select_blocks(t(ref, dev), bt, ctx, 16, ms, sinks, recents)
        assert fbt.dtype == itype and fcl.dtype == itype and tuple(fbt.shape) == (3, ms)
        assert np.array_equal(fcl.cpu().numpy(), bsel[f"sel_fcl_{tag}"])
        k = min(ms, 100)
        for s in range(3):
            m = min(k, int(nb[s]))
            assert np.array_equal(fbt[s, :m].cpu().numpy(), bsel[f"sel_fbt_{tag}"][s, :m])
        assert torch.all(fbt[:, k:] == 0)
        # and column for column like the oracle (which fixes the order among equal keys the same way)
        obt, ocl = O.block_select(ref, bsel["sel_bt"], bsel["sel_ctx"], 16, ms, sinks, recents)
        assert np.array_equal(fbt.cpu().numpy(), obt) and np.array_equal(fcl.cpu().numpy(), ocl)


def test_selector_class_and_large_table(bsel, dev):
    sel = BlockSelector(300, 2, 64, dev, t(bsel["centroids"], dev), select_ratio=0.1)
    assert sel.max_selected == int(bsel["cls_max_selected"])
    sel._rep_cache.rep_even.copy_(t(bsel["sel_rep_even"], dev))
    sel._rep_cache.rep_odd.copy_(t(bsel["sel_rep_odd"], dev))
    fbt, fcl = sel.select(t(bsel["sel_q_even"], dev), t(bsel["sel_q_odd"], dev), t(bsel["sel_bt"], dev), t(bsel["sel_ctx"], dev), 4, 16)
    assert np.array_equal(fcl.cpu().numpy(), bsel["cls_fcl"])
    nb = (bsel["sel_ctx"] + 15) // 16
    for s in range(3):
        m = min(30, int(nb[s]))
        assert np.array_equal(fbt[s, :m].cpu().numpy(), bsel["cls_fbt"][s, :m])
    # disabled selector and short tables pass the inputs through
    off = BlockSelector(300, 2, 64, dev, t(bsel["centroids"], dev))
    bt = t(bsel["sel_bt"], dev)
    assert off.select(None, None, bt, None, 4)[0] is bt
    assert sel.select(None, None, bt[:, :32], t(bsel["sel_ctx"], dev), 4)[0].shape[1] == 32
    # a wide table with many equal scores: 20,000 columns, scores quantised to 64 levels
    rng = np.random.default_rng(3)
    S, B = 4, 20000
    scores = np.round(rng.standard_normal((S, B)) * 8).astype(np.float32) / 8
    ctx = np.array([B * 16, B * 16 - 7, 5000 * 16 + 3, 16], dtype=np.int64)
    table = rng.integers(0, 1 << 20, size=(S, B)).astype(np.int64)
    for ms in (7, 2000, 25000):
        fbt, fcl = select_blocks(t(scores, dev), t(table, dev), t(ctx, dev), 16, ms)
        obt, ocl = O.block_select(scores, table, ctx, 16, ms)
        assert np.array_equal(fbt.cpu().numpy(), obt) and np.array_equal(fcl.cpu().numpy(), ocl)


def test_selection_with_signed_zeros_and_nan_scores(dev):
    """Scores quantised to a few levels hold both zeros: they are equal keys (the lower column wins, as between
    any equal scores); a NaN ranks above everything (torch.topk's order, block_selector.py:205-207)."""
    rng = np.random.default_rng(11)
    S, B = 6, 300
    sc = (np.round(rng.standard_normal((S, B)) * 3) / 3).astype(np.float32)
    assert np.any(np.signbit(sc) & (sc == 0)) and np.any(~np.signbit(sc) & (sc == 0))
    sc[rng.random((S, B)) < 0.02] = np.nan
    sc[0, 5] = -np.nan
    ctx = np.array([B * 16, B * 16 - 5, 40 * 16, 1, 0, 150 * 16 + 1], dtype=np.int64)
    table = rng.integers(0, 1 << 20, size=(S, B)).astype(np.int64)
    nb = (ctx + 15) // 16
    for ms, sinks, recents in ((30, 2, 2), (7, 0, 0), (100, 3, 1), (B + 4, 1, 1)):
        fbt, fcl = select_blocks(t(sc, dev), t(table, dev), t(ctx, dev), 16, ms, sinks, recents)
        obt, ocl = O.block_select(sc, table, ctx, 16, ms, sinks, recents)
        assert np.array_equal(fcl.cpu().numpy(), ocl)
        k = min(ms, B)
        for s in range(S):
            m = min(k, int(nb[s]))
            assert np.array_equal(fbt[s, :m].cpu().numpy(), obt[s, :m]), (ms, s)


def test_sparse_attention_end_to_end(golden, dev):
    """Encode -> representatives -> selection -> attention equals attention over the selected blocks alone."""
    tq = akv.TurboQuant(head_dim=128, bits=4, device=str(dev))
    tq.rotation = torch.from_numpy(golden["rotation_d128_seed42"]).to(dev)
    rng = np.random.default_rng(9)
    S, QH, KVH, BS, NBLK, BPS = 2, 8, 2, 16, 200, 80
    ctx = np.array([80 * BS - 3, 70 * BS], dtype=np.int64)
    k = t(kv_like(rng, (NBLK, BS, KVH, 128)), dev)
    v = t(kv_like(rng, (NBLK, BS, KVH, 128)), dev)
    kp, kn = tq.encode(k)
    vp, vn = tq.encode(v)
    table = np.stack([rng.permutation(NBLK)[:BPS] for _ in range(S)]).astype(np.int64)
    sel = BlockSelector(NBLK, KVH, 64, dev, tq.centroids, select_ratio=0.1, min_blocks_for_selection=64)
    blk = torch.arange(NBLK, device=dev).repeat_interleave(BS)
    sel.update_reps(blk, torch.arange(BS, device=dev).repeat(NBLK), kp.reshape(NBLK * BS, KVH, 64), kn.reshape(NBLK * BS, KVH))
    # representatives against the oracle
    acc_e = np.zeros((NBLK, KVH, 64), np.float32); acc_o = np.zeros_like(acc_e); cnt = np.zeros((NBLK, KVH), np.int32)
    O.block_rep_update(acc_e, acc_o, cnt, blk.cpu().numpy(), kp.reshape(-1, KVH, 64).cpu().numpy(), kn.reshape(-1, KVH).cpu().numpy(),
                       tq.centroids.cpu().numpy())
    np.testing.assert_allclose(sel._rep_cache.rep_even.cpu().numpy(), acc_e / 16, rtol=1e-5, atol=1e-6)
    q = torch.from_numpy(rng.standard_normal((S, QH, 128)).astype(np.float32)).to(dev).half()
    sparse = akv.TQPagedAttention(tq, QH, block_selector=sel)
    dense = akv.TQPagedAttention(tq, QH)
    out = sparse.forward(q, kp, kn, vp, vn, t(table, dev), t(ctx, dev), block_size=BS, num_kv_heads=KVH)
    q_rot = q.float() @ tq.rotation.T
    fbt, fcl = sel.select(q_rot[..., 0::2].contiguous(), q_rot[..., 1::2].contiguous(), t(table, dev), t(ctx, dev), QH // KVH, BS)
    assert tuple(fbt.shape) == (S, 20) and torch.all(fcl == 20 * BS)
    want = dense.forward(q, kp, kn, vp, vn, fbt, fcl, block_size=BS, num_kv_heads=KVH)
    assert torch.equal(out, want)
    # the first two and the last two blocks of every sequence are always among the selected
    for s in range(S):
        nb = (int(ctx[s]) + BS - 1) // BS
        chosen = set(fbt[s].cpu().tolist())
        assert {int(table[s, 0]), int(table[s, 1]), int(table[s, nb - 2]), int(table[s, nb - 1])} <= chosen

"""tq25 hybrid codec and attention (HIP) against the reference's vectors and the oracle."""
import math

import numpy as np
import pytest
import torch

import aitherkvcache_amd as akv
from oracle import tq_oracle as O
from tests.util import kv_like, MAX_ULPS

pytestmark = pytest.mark.gpu
ROW = 44


def t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def params(tq25):
    books = ((tq25["g0_centroids"], tq25["g0_boundaries"]), (tq25["g1_centroids"], tq25["g1_boundaries"]))
    return O.HybridParams(tq25["g0_had"], tq25["g1_had"], tq25["g0_qjl"], tq25["g1_qjl"], codebooks=books, mode="tq25")


def compare_rows(got, ref):
    """Rows must agree byte for byte, except that a norm whose float32 value sits on an fp16 rounding boundary
    may land one fp16 step away (sum order), and a code / sign whose rotated value sits on a decision boundary
    may flip.  Returns counts of each kind."""
    got, ref = got.reshape(-1, ROW), ref.reshape(-1, ROW)
    bad_rows = np.where(np.any(got != ref, axis=1))[0]
    stats = {"rows": len(got), "rows_differing": len(bad_rows), "norm_ulp": 0, "code_bytes": 0, "sign_bytes": 0}
    for r in bad_rows:
        for lo in (12, 14, 40, 42):
            a = int(got[r, lo]) | int(got[r, lo + 1]) << 8
            b = int(ref[r, lo]) | int(ref[r, lo + 1]) << 8
            if a != b:
                assert abs(a - b) == 1, (r, lo, a, b)            # one fp16 step at most
                stats["norm_ulp"] += 1
        stats["code_bytes"] += int(np.sum(got[r, 0:8] != ref[r, 0:8]) + np.sum(got[r, 16:28] != ref[r, 16:28]))
        stats["sign_bytes"] += int(np.sum(got[r, 8:12] != ref[r, 8:12]) + np.sum(got[r, 28:40] != ref[r, 28:40]))
    return stats


def test_golden_encode_decode(tq25, dev):
    h = akv.HybridTurboQuant(head_dim=128, mode="tq25", device=str(dev))
    h.calibrate_uniform()
    packed = h.encode(t(tq25["x"], dev))
    assert packed.dtype == torch.uint8 and packed.shape == (48, ROW)
    st = compare_rows(packed.cpu().numpy(), tq25["packed"])
    print("[tq25 golden]", st)
    assert st["rows_differing"] <= 2
    dec = h.decode(t(tq25["packed"], dev))
    assert dec.dtype == torch.float32
    assert np.array_equal(dec.cpu().numpy(), tq25["decoded"])            # bit-exact
    h2 = akv.HybridTurboQuant(mode="tq25", device=str(dev))
    h2.calibrate_uniform(num_kv_heads=2)
    p2 = h2.encode(t(tq25["x_heads2"], dev))
    assert p2.shape == (5, 2, ROW)
    assert compare_rows(p2.cpu().numpy(), tq25["packed_heads2"])["rows_differing"] <= 1
    assert np.array_equal(h2.decode(t(tq25["packed_heads2"], dev)).cpu().numpy(), tq25["decoded_heads2"])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_encode_vs_oracle_bulk(tq25, dev, dtype):
    h = akv.HybridTurboQuant(mode="tq25", device=str(dev))
    h.calibrate_uniform()
    hp = params(tq25)
    rng = np.random.default_rng(9)
    x = t(kv_like(rng, (20000, 128), np.float32), dev).to(dtype)
    x[5] = 0
    x[6, :32] = 0
    packed = h.encode(x).cpu().numpy()
    ref = O.hybrid_encode(x.float().cpu().numpy(), hp)
    st = compare_rows(packed, ref)
    # every bit that differs from a float64 evaluation must sit within MAX_ULPS float32 ulps of its flip
    # point (codes: rotated value against the boundary; signs: projection against zero, with the row's own
    # codes); stored norms at most one fp16 step from the rounded float64 norm
    m = O.hybrid_encode_margins(x.float().cpu().numpy(), packed, hp)
    worst = {k: max(float(np.abs(v[g]).max()) for g in (0, 1)) for k, v in m.items()}
    flips = {k: sum(int((v[g] != 0).sum()) for g in (0, 1)) for k, v in m.items()}
    print("[tq25 bulk]", dtype, st, "worst", worst, "flips", flips)
    assert worst["code_ulps"] <= MAX_ULPS and worst["sign_ulps"] <= MAX_ULPS
    assert worst["norm_steps"] <= 1 and worst["rnorm_steps"] <= 1
    assert st["rows_differing"] <= 60
    assert st["code_bytes"] + st["sign_bytes"] <= 80
    # decode is exact integer/butterfly work
    dec = h.decode(t(ref, dev)).cpu().numpy()
    assert np.array_equal(dec, O.hybrid_decode(ref, hp))
    assert h.decode(t(ref, dev)[:0]).shape == (0, 128)
    # strided rows in and out
    wide = torch.zeros(100, 200, dtype=dtype, device=dev)
    wide[:, :128] = x[:100]
    assert np.array_equal(h.encode(wide[:, :128]).cpu().numpy(), packed[:100])
    rep = h.validate(4000)
    assert rep["packed_dim_bytes"] == ROW and rep["cosine_similarity"] > 0.8


def build_cache(rng, h, dev, NB, KVH, BS=16, row=ROW):
    kc = torch.zeros(NB, BS, KVH, row, dtype=torch.uint8, device=dev)
    vc = torch.zeros_like(kc)
    keys, vals = kv_like(rng, (NB * BS, KVH, 128)), kv_like(rng, (NB * BS, KVH, 128))
    slots = torch.arange(NB * BS, device=dev)
    akv.hybrid_encode_and_store(h, t(keys, dev), slots, kc, BS)
    akv.hybrid_encode_and_store(h, t(vals, dev), slots, vc, BS)
    return kc, vc, keys, vals


@pytest.mark.parametrize("qh,kvh", [(32, 8), (6, 2)])
def test_paged_attention_vs_oracle(tq25, dev, qh, kvh):
    h = akv.HybridTurboQuant(mode="tq25", device=str(dev))
    h.calibrate_uniform(num_kv_heads=kvh)
    hp = params(tq25)
    rng = np.random.default_rng(21 + qh)
    NB = 64
    kc, vc, keys, _ = build_cache(rng, h, dev, NB, kvh)
    # paged write == flat encode of the same vectors
    assert torch.equal(kc.reshape(-1, kvh, ROW), h.encode(t(keys, dev)))
    ctx = np.array([0, 1, 16, 17, 500, 333], dtype=np.int64)
    tables = np.full((6, 32), -3, dtype=np.int64)
    for s, c_ in enumerate(ctx):
        nb = -(-int(c_) // 16)
        tables[s, :nb] = rng.permutation(NB)[:nb]
    q = rng.standard_normal((6, qh, 128)).astype(np.float16)
    scale = 1 / math.sqrt(128)
    attn = akv.HybridPagedAttention(h, qh)
    out = attn.forward(t(q, dev), kc, vc, t(tables, dev), t(ctx, dev), scale=scale)
    assert out.dtype == torch.float16
    ref = O.hybrid_paged_attention(q, kc.cpu().numpy(), vc.cpu().numpy(), tables, ctx, hp, scale, dtype=np.float64)
    got = out.cpu().numpy().astype(np.float64)
    print(f"[tq25 attn] qh={qh} max|diff|={np.max(np.abs(got - ref)):.2e}")
    # 2e-3 plus half an fp16 ulp of the output itself where outputs are large
    assert np.all(got[0] == 0) and np.all(np.abs(got - ref) <= 2e-3 + 2.0 ** -11 * np.abs(ref))
    o32 = attn.forward(t(q.astype(np.float32), dev), kc, vc, t(tables, dev).int(), t(ctx, dev).int(), scale=0.05)
    ref32 = O.hybrid_paged_attention(q, kc.cpu().numpy(), vc.cpu().numpy(), tables, ctx, hp, 0.05, dtype=np.float64)
    assert np.max(np.abs(o32.cpu().numpy() - ref32)) <= 2e-4


@pytest.mark.parametrize("qh,kvh,bs", [(32, 8, 16), (12, 1, 16), (8, 2, 32), (4, 4, 16), (16, 2, 8)])
def test_paged_attention_ragged_batch_with_stale_rows(tq25, dev, qh, kvh, bs):
    """Ragged contexts, permuted tables with padding entries, rows wider than the packed vector, and stale
    data in every position past a context: the result is the oracle's for the addressed tokens only."""
    h = akv.HybridTurboQuant(mode="tq25", device=str(dev))
    h.calibrate_uniform(num_kv_heads=kvh)
    hp = params(tq25)
    rng = np.random.default_rng(100 + qh + bs)
    NB = 96
    kc, vc, _, _ = build_cache(rng, h, dev, NB, kvh, BS=bs, row=48)
    ctx = np.array([3 * bs + 5, 0, bs, 1, 11 * bs, 7 * bs - 1, 2], dtype=np.int64)
    S, W = len(ctx), 12
    tables = np.full((S, W), 10 ** 6, dtype=np.int64)          # padding entries far outside the cache
    for s, c_ in enumerate(ctx):
        nb = -(-int(c_) // bs)
        tables[s, :nb] = rng.permutation(NB)[:nb]
    q = rng.standard_normal((S, qh, 128)).astype(np.float32)
    attn = akv.HybridPagedAttention(h, qh)
    out = attn.forward(t(q, dev), kc, vc, t(tables, dev), t(ctx, dev), block_size=bs, scale=0.09)
    ref = O.hybrid_paged_attention(q, kc.cpu().numpy()[..., :ROW], vc.cpu().numpy()[..., :ROW],
                                   np.where(tables >= NB, 0, tables), ctx, hp, 0.09, block_size=bs, dtype=np.float64)
    err = np.max(np.abs(out.cpu().numpy() - ref))
    print(f"[tq25 ragged] qh={qh} kvh={kvh} bs={bs} max|diff|={err:.2e}")
    assert err <= 2e-4 and np.all(out.cpu().numpy()[1] == 0)
    assert attn.last_call_status() == 0


def test_hybrid_decode_step_with_tq25(tq25, dev):
    """tq::hybrid_decode_step's body (vllm/hooks.py:240-345) with a tq25 quantizer: the new token is written, the
    attention covers it."""
    from aitherkvcache_amd.vllm import hooks
    hp = params(tq25)
    rng = np.random.default_rng(77)
    KVH, QH, BS, NB, S = 2, 8, 16, 12, 3
    h = akv.HybridTurboQuant(mode="tq25", device=str(dev))
    h.calibrate_uniform(num_kv_heads=KVH)
    saved = dict(hooks._tq_quantizers), dict(hooks._tq_fused_attn)
    try:
        hooks._tq_quantizers[128] = h
        hooks._tq_fused_attn.clear()
        kv = torch.zeros(NB, 2, BS, KVH, ROW, dtype=torch.uint8, device=dev)
        hist_k, hist_v = kv_like(rng, (NB * BS, KVH, 128)), kv_like(rng, (NB * BS, KVH, 128))
        akv.hybrid_encode_and_store(h, t(hist_k, dev), torch.arange(NB * BS, device=dev), kv[:, 0], BS)
        akv.hybrid_encode_and_store(h, t(hist_v, dev), torch.arange(NB * BS, device=dev), kv[:, 1], BS)
        ctx = np.array([20, 1, 33], dtype=np.int64)                  # lengths that include the new token
        tables = np.stack([rng.permutation(NB)[:4] for _ in range(S)]).astype(np.int64)
        slots = np.array([tables[s, (c - 1) // BS] * BS + (c - 1) % BS for s, c in enumerate(ctx)], dtype=np.int64)
        key, val = kv_like(rng, (S, KVH, 128)), kv_like(rng, (S, KVH, 128))
        q = rng.standard_normal((S, QH, 128)).astype(np.float16)
        out = torch.zeros(S, QH, 128, dtype=torch.float16, device=dev)
        res = hooks.hybrid_decode_step(t(q, dev), t(key, dev), t(val, dev), kv, out, t(slots, dev), t(tables, dev),
                                       t(ctx, dev), 0, QH, KVH, 128, 0.1, S)
        kc, vc = kv[:, 0].cpu().numpy(), kv[:, 1].cpu().numpy()
        for s in range(S):
            blk, pos = divmod(int(slots[s]), BS)
            st = compare_rows(kc[blk, pos], O.hybrid_encode(key[s], hp))
            assert st["code_bytes"] + st["sign_bytes"] == 0
        ref = O.hybrid_paged_attention(q, kc, vc, tables, ctx, hp, 0.1, dtype=np.float64)
        got = res.cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - ref) <= 2e-3 + 2.0 ** -11 * np.abs(ref))
    finally:
        hooks._tq_quantizers.clear(); hooks._tq_quantizers.update(saved[0])
        hooks._tq_fused_attn.clear(); hooks._tq_fused_attn.update(saved[1])


def test_ranked_calibration_is_the_codec_on_permuted_coordinates(tq25, dev):
    """calibrate(sample): per head the 32 coordinates of largest mean square form group 0.  Encoding a vector
    is encoding its coordinates in group order with the uniform split, decoding scatters them back."""
    rng = np.random.default_rng(5)
    KVH = 2
    sample = rng.standard_normal((256, KVH, 128)).astype(np.float32) * (1.0 + 3.0 * (rng.random((1, KVH, 128)) > 0.7))
    h = akv.HybridTurboQuant(mode="tq25", device=str(dev))
    h.calibrate(t(sample, dev))
    order = h.group_order.cpu().numpy()
    assert order.shape == (KVH, 128) and all(sorted(order[k]) == list(range(128)) for k in range(KVH))
    u = akv.HybridTurboQuant(mode="tq25", device=str(dev))
    u.calibrate_uniform(num_kv_heads=KVH)
    x = kv_like(rng, (50, KVH, 128), np.float32)
    xp = np.stack([x[:, k, order[k]] for k in range(KVH)], axis=1)
    p = h.encode(t(x, dev))
    assert torch.equal(p, u.encode(t(xp, dev)))
    back = h.decode(p).cpu().numpy()
    ub = u.decode(p).cpu().numpy()
    for k in range(KVH):
        assert np.array_equal(back[:, k, order[k]], ub[:, k])


@pytest.mark.parametrize("mode,row", [("tq35", 64), ("tq25", 44)])
def test_key_and_value_of_a_step_in_one_call(golden, tq25, dev, mode, row):
    """hybrid_encode_and_store_pair: K and V of a step by one call -- the same bytes as two single calls, for a
    small step (one launch), a large one (the form for large calls, twice), skipped slots, pitched caches, and
    tensors whose strides differ (two single calls underneath)."""
    h = akv.HybridTurboQuant(mode=mode, device=str(dev))
    h.calibrate_uniform(num_kv_heads=4)
    rng = np.random.default_rng(61)
    KVH, BS = 4, 16
    for T, NB in ((1, 4), (37, 8), (300, 24), (5000, 320)):
        k, v = t(kv_like(rng, (T, KVH, 128)), dev), t(kv_like(rng, (T, KVH, 128)), dev)
        slots = rng.permutation(NB * BS)[:T].astype(np.int64)
        slots[::13] = -1
        sd = t(slots, dev)
        kv = torch.full((NB, 2, BS, KVH, row + 4), 0xAB, dtype=torch.uint8, device=dev)      # the serving layout
        akv.hybrid_encode_and_store_pair(h, k, v, sd, kv[:, 0, :, :, :row], kv[:, 1, :, :, :row], BS)
        ref = torch.full_like(kv, 0xAB)
        akv.hybrid_encode_and_store(h, k, sd, ref[:, 0, :, :, :row], BS)
        akv.hybrid_encode_and_store(h, v, sd, ref[:, 1, :, :, :row], BS)
        assert torch.equal(kv, ref), (mode, T)
    wide = torch.zeros(37, KVH, 136, dtype=k.dtype, device=dev)
    k37, v37 = k[:37].contiguous(), v[:37]
    wide[..., :128] = v37
    a = torch.zeros(8, BS, KVH, row, dtype=torch.uint8, device=dev)
    b = torch.zeros_like(a)
    sl = torch.arange(37, device=dev)
    akv.hybrid_encode_and_store_pair(h, k37, wide[..., :128], sl, a, b, BS)
    assert torch.equal(a.reshape(-1, KVH, row)[:37], h.encode(k37)) and torch.equal(b.reshape(-1, KVH, row)[:37], h.encode(v37))

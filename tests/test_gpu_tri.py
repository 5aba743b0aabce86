"""TriAttention decode_step (HIP) against the reference's outputs and the oracle."""
import numpy as np
import pytest
import torch

from aitherkvcache_amd.triattention import TriAttention, TriAttentionConfig, SpectralEncoding
from oracle import tq_oracle as O

pytestmark = pytest.mark.gpu
TOL = 2e-5     # float32 outputs; differences come from sin/cos last-place and summation order


def t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def enc(golden, nm, dev):
    return SpectralEncoding(t(golden[f"tri_{nm}_indices"], dev), t(golden[f"tri_{nm}_packed"], dev),
                            t(golden[f"tri_{nm}_scales"], dev))


def test_golden_decode_step(golden, dev):
    cfg = TriAttentionConfig(head_dim=128, num_freqs=12, coeff_bits=4, num_kv_heads=2, num_query_heads=8,
                             rope_base=1_000_000.0)
    tri = TriAttention(cfg, device=str(dev))
    assert np.array_equal(tri._theta.cpu().numpy(), golden["theta_d128_base1e6"])
    ke, ve = enc(golden, "k", dev), enc(golden, "v", dev)
    q = t(golden["tri_q"], dev)
    out = tri.decode_step(q, ke, ve)
    assert out.dtype == torch.float32 and out.shape == (2, 8, 128)
    e1 = np.max(np.abs(out.cpu().numpy() - golden["tri_out_default_pos"]))
    out2 = tri.decode_step(q, ke, ve, t(golden["tri_qpos"], dev), t(golden["tri_kpos"], dev))
    e2 = np.max(np.abs(out2.cpu().numpy() - golden["tri_out_explicit_pos"]))
    print(f"[tri golden] default-pos {e1:.2e}, explicit-pos {e2:.2e}")
    assert e1 <= TOL and e2 <= TOL
    # int32 positions, fp16 query
    out3 = tri.decode_step(q.half(), ke, ve, t(golden["tri_qpos"], dev).int(), t(golden["tri_kpos"], dev).int())
    ref3 = O.tri_decode_step(golden["tri_q"].astype(np.float16), tuple(golden[f"tri_k_{n}"] for n in ("indices", "packed", "scales")),
                             tuple(golden[f"tri_v_{n}"] for n in ("indices", "packed", "scales")),
                             golden["theta_d128_base1e6"], golden["tri_qpos"], golden["tri_kpos"])
    assert np.max(np.abs(out3.cpu().numpy() - ref3)) <= TOL


@pytest.mark.parametrize("B,S,QH,KVH,D,F,base", [(3, 1000, 32, 8, 128, 12, 1e6), (2, 333, 6, 2, 32, 4, 1e4),
                                                 (1, 64, 4, 4, 64, 32, 1e4), (2, 5000, 8, 1, 128, 12, 1e6),
                                                 (2, 700, 8, 2, 128, 20, 1e6), (1, 1500, 16, 16, 128, 12, 1e6),
                                                 (2, 130, 12, 4, 128, 12, 1e4)])
def test_vs_oracle_shapes(dev, B, S, QH, KVH, D, F, base):
    cfg = TriAttentionConfig(head_dim=D, num_freqs=F, coeff_bits=4, num_kv_heads=KVH, num_query_heads=QH, rope_base=base)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(S)
    pair_std = (np.arange(D // 2) + 1.0) ** -0.75
    keys = (rng.standard_normal((B, S, KVH, D // 2, 2)) * pair_std[:, None]).reshape(B, S, KVH, D).astype(np.float16)
    vals = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    k_enc, v_enc = tri.encode_kv(t(keys, dev), t(vals, dev))
    # the write side (torch ops on the device) agrees with the oracle's encoder
    ki, kpk, ks = O.spectral_encode(keys, F)
    assert np.array_equal(k_enc.indices.cpu().numpy(), ki) and np.array_equal(k_enc.packed.cpu().numpy(), kpk)
    assert np.array_equal(k_enc.scales.cpu().numpy(), ks)
    q = rng.standard_normal((B, QH, D)).astype(np.float32)
    qpos = rng.integers(S, 40000, size=B)
    kpos = np.sort(rng.integers(0, 32768, size=(B, S)), axis=-1)
    theta = tri._theta.cpu().numpy()
    out = tri.decode_step(t(q, dev), k_enc, v_enc, t(qpos, dev), t(kpos, dev)).cpu().numpy()
    ref = O.tri_decode_step(q, (ki, kpk, ks), tuple(x.cpu().numpy() for x in v_enc), theta, qpos, kpos)
    err = np.max(np.abs(out - ref))
    print(f"[tri] B={B} S={S} D={D} F={F} max|diff|={err:.2e} max|out|={np.abs(ref).max():.3f}")
    assert err <= TOL
    out_d = tri.decode_step(t(q, dev), k_enc, v_enc).cpu().numpy()
    ref_d = O.tri_decode_step(q, (ki, kpk, ks), tuple(x.cpu().numpy() for x in v_enc), theta)
    assert np.max(np.abs(out_d - ref_d)) <= TOL


def test_config4_literal_shape(dev):
    """The benchmark shape itself: batch 8 x 32,768 tokens, 32 query / 8 kv heads, d = 128, F = 12 int4,
    keys with a power-law pair spectrum (seed 4).  One batch element against the oracle (its encoder and
    its decode_step), and for the whole batch: every element computed alone equals its row of the batched
    call, and elements given the same cache rows and query produce the same output."""
    cfg = TriAttentionConfig(head_dim=128, num_freqs=12, coeff_bits=4, num_kv_heads=8, num_query_heads=32, rope_base=1e6)
    tri = TriAttention(cfg, device=str(dev))
    B, S = 8, 32768
    g = torch.Generator(device=dev).manual_seed(4)
    std = (torch.arange(64, device=dev) + 1.0) ** -0.75
    keys = (torch.randn(B, S, 8, 64, 2, device=dev, generator=g) * std[:, None]).reshape(B, S, 8, 128).half()
    vals = torch.randn(B, S, 8, 128, device=dev, generator=g).half()
    keys[7], vals[7] = keys[2], vals[2]                      # element 7 repeats element 2
    q = torch.randn(B, 32, 128, device=dev, generator=g)
    q[7] = q[2]
    k_enc, v_enc = tri.encode_kv(keys, vals)
    out = tri.decode_step(q, k_enc, v_enc)
    assert out.shape == (B, 32, 128) and torch.isfinite(out).all()
    assert torch.equal(out[7], out[2])
    for b in (0, 5):
        one = tri.decode_step(q[b:b + 1], SpectralEncoding(*(x[b:b + 1] for x in k_enc)),
                              SpectralEncoding(*(x[b:b + 1] for x in v_enc)))
        assert torch.max(torch.abs(one[0] - out[b])).item() <= TOL      # the split count may differ
    b = 3
    ke = O.spectral_encode(keys[b:b + 1].cpu().numpy(), 12)
    ve = O.spectral_encode(vals[b:b + 1].cpu().numpy(), 12)
    for got, want in zip(tuple(k_enc) + tuple(v_enc), ke + ve):
        assert np.array_equal(got[b:b + 1].cpu().numpy(), want)
    ref = O.tri_decode_step(q[b:b + 1].cpu().numpy(), ke, ve, tri._theta.cpu().numpy())
    err = np.max(np.abs(out[b:b + 1].cpu().numpy() - ref))
    print(f"[tri config 4] element {b}: max|diff|={err:.2e} max|out|={np.abs(ref).max():.3f}")
    assert err <= TOL


def test_uniform_values_property(dev):
    """Every token holds the same value row -> the output is that row, whatever the scores
    (softmax weights sum to one across all splits)."""
    cfg = TriAttentionConfig(num_kv_heads=8, num_query_heads=32)
    tri = TriAttention(cfg, device=str(dev))
    B, S = 2, 32768
    g = torch.Generator(device=dev).manual_seed(4)
    keys = torch.randn(B, S, 8, 128, device=dev, generator=g).half()
    one = torch.randn(1, 1, 8, 128, device=dev, generator=g).half()
    k_enc, _ = tri.encode_kv(keys, keys)
    v1 = tri.encoder.encode(one)
    v_enc = SpectralEncoding(v1.indices.expand(B, S, 8, 12).contiguous(), v1.packed.expand(B, S, 8, 12).contiguous(),
                             v1.scales.expand(B, S, 8).contiguous())
    q = torch.randn(B, 32, 128, device=dev, generator=g)
    out = tri.decode_step(q, k_enc, v_enc)
    want = tri.encoder.decode(v1).reshape(1, 8, 1, 128).expand(B, 8, 4, 128).reshape(B, 32, 128)
    assert torch.max(torch.abs(out - want)).item() <= 1e-5


def test_spectral_encode_golden(golden, dev):
    """The write-side kernel reproduces the reference's encodings of the golden keys and values byte for byte."""
    tri = TriAttention(TriAttentionConfig(num_kv_heads=2, num_query_heads=8), device=str(dev))
    for nm, src in (("k", "tri_keys"), ("v", "tri_vals")):
        e = tri.encoder.encode(t(golden[src], dev))
        assert e.indices.dtype == torch.uint8 and e.packed.dtype == torch.uint8 and e.scales.dtype == torch.float16
        assert np.array_equal(e.indices.cpu().numpy(), golden[f"tri_{nm}_indices"])
        assert np.array_equal(e.packed.cpu().numpy(), golden[f"tri_{nm}_packed"])
        assert np.array_equal(e.scales.cpu().numpy(), golden[f"tri_{nm}_scales"])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("D,F", [(128, 12), (64, 7), (32, 16)])
def test_spectral_encode_vs_oracle(dev, dtype, D, F):
    rng = np.random.default_rng(D + F)
    n = 5000
    x = (rng.standard_normal((n, D)) * rng.lognormal(0, 1.0, (n, 1))).astype(np.float32)
    x[7] = 0.0                                  # all energies equal: the lowest indices are kept, scale 1e-8 -> fp16 0
    x[8, 2:] = 0.0                              # fewer non-zero pairs than F
    x[9] *= 1e-6
    xt = torch.from_numpy(x).to(dev).to(dtype)
    cfg = TriAttentionConfig(head_dim=D, num_freqs=F, num_kv_heads=1, num_query_heads=1)
    tri = TriAttention(cfg, device=str(dev))
    e = tri.encoder.encode(xt)
    ri, rp, rs = O.spectral_encode(xt.float().cpu().numpy(), F)
    assert np.array_equal(e.indices.cpu().numpy(), ri)
    assert np.array_equal(e.packed.cpu().numpy(), rp)
    assert np.array_equal(e.scales.cpu().numpy(), rs)
    # batch shapes and the empty batch
    e2 = tri.encoder.encode(xt[:24].reshape(2, 3, 4, D))
    assert e2.indices.shape == (2, 3, 4, F) and e2.scales.shape == (2, 3, 4)
    assert torch.equal(e2.indices.reshape(24, F), e.indices[:24])
    e0 = tri.encoder.encode(xt[:0])
    assert e0.indices.shape == (0, F)


@pytest.mark.parametrize("bits", [4, 8])
def test_spectral_encode_energies_a_rounding_apart(dev, bits):
    """float32 pairs on the unit circle: every energy is 1 up to the last places, so which pairs are kept
    depends on each square and their sum being rounded on its own, as the reference's pow(2).sum(-1) does
    (a fused multiply-add moves the result by a place and changes the selection)."""
    D, F, n = 128, 12, 20000
    rng = np.random.default_rng(77 + bits)
    ang = rng.uniform(0, 2 * np.pi, (n, D // 2))
    x = np.stack([np.cos(ang), np.sin(ang)], -1).astype(np.float32).reshape(n, D)
    x *= np.float32(2.0) ** rng.integers(-3, 4, (n, 1)).astype(np.float32)       # exact scalings of whole rows
    a, b = x[:, 0::2].astype(np.float64), x[:, 1::2].astype(np.float64)
    plain = (x[:, 0::2] * x[:, 0::2] + x[:, 1::2] * x[:, 1::2]).astype(np.float32)
    fused = (a * a + (x[:, 1::2] * x[:, 1::2]).astype(np.float64)).astype(np.float32)
    assert np.mean(plain != fused) > 0.05                  # the case is present in the data
    xt = torch.from_numpy(x).to(dev)
    tri = TriAttention(TriAttentionConfig(head_dim=D, num_freqs=F, coeff_bits=bits, num_kv_heads=1, num_query_heads=1),
                       device=str(dev))
    e = tri.encoder.encode(xt)
    ri, rp, rs = O.spectral_encode(x, F, bits)
    assert np.array_equal(e.indices.cpu().numpy(), ri)
    assert np.array_equal(e.packed.cpu().numpy(), rp)
    assert np.array_equal(e.scales.cpu().numpy(), rs)


@pytest.mark.parametrize("KVH,QH,bt_dtype,BS", [(8, 32, torch.int32, 16), (2, 8, torch.int64, 16), (4, 4, torch.int32, 16),
                                                 (8, 32, torch.int64, 32), (1, 4, torch.int32, 8), (16, 16, torch.int32, 16),
                                                 (8, 32, torch.int32, 24), (2, 8, torch.int64, 3), (4, 16, torch.int32, 100),
                                                 (8, 8, torch.int32, 1)])
def test_paged_decode_vs_oracle(dev, KVH, QH, bt_dtype, BS):
    """decode_step_paged over a block pool with permuted block tables, ragged context lengths (one
    empty, one ending inside a block, one filling its table) against the oracle's fetch + decode and
    against fetch_sequence + decode_step on the device."""
    from aitherkvcache_amd.triattention import SpectralKVCache
    cfg = TriAttentionConfig(num_kv_heads=KVH, num_query_heads=QH, block_size=BS)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(100 + KVH)
    D = 128
    lens = [0, 1, 777, 2048, 1500]
    B, max_bps = len(lens), -(-2048 // BS)        # (block sizes that are no power of two among them)
    NB = 6400 // BS + 8
    cache = SpectralKVCache(cfg, max_blocks=NB, device=str(dev))
    perm = rng.permutation(NB)
    tables = np.full((B, max_bps), -7, dtype=np.int64)        # padding entries are never dereferenced
    used = 0
    pair_std = (np.arange(D // 2) + 1.0) ** -0.75
    for b, n in enumerate(lens):
        nb = -(-n // BS)
        tables[b, :nb] = perm[used:used + nb]
        used += nb
        if n == 0:
            continue
        keys = (rng.standard_normal((1, n, KVH, D // 2, 2)) * pair_std[:, None]).reshape(1, n, KVH, D).astype(np.float16)
        vals = rng.standard_normal((1, n, KVH, D)).astype(np.float16)
        k_enc, v_enc = tri.encode_kv(t(keys, dev), t(vals, dev))
        cache.store_sequence(torch.from_numpy(tables[b]), SpectralEncoding(*(x[0] for x in k_enc)),
                             SpectralEncoding(*(x[0] for x in v_enc)))
    q = rng.standard_normal((B, QH, D)).astype(np.float32)
    bt = torch.from_numpy(tables).to(dev).to(bt_dtype)
    cl = torch.tensor(lens, device=dev, dtype=torch.int32)
    out = tri.decode_step_paged(t(q, dev), cache, bt, cl).cpu().numpy()
    arrays = [x.cpu().numpy() for x in cache._arrays()]
    ref = O.tri_decode_step_paged(q, arrays, tables, lens, BS, tri._theta.cpu().numpy())
    err = np.max(np.abs(out - ref))
    print(f"[tri paged] KVH={KVH} max|diff|={err:.2e}")
    assert err <= TOL and not np.any(out[0])
    qpos = np.array([5, 9, 3000, 40000, 1501])
    out_q = tri.decode_step_paged(t(q, dev), cache, bt, cl, t(qpos, dev)).cpu().numpy()
    ref_q = O.tri_decode_step_paged(q, arrays, tables, lens, BS, tri._theta.cpu().numpy(), qpos)
    assert np.max(np.abs(out_q - ref_q)) <= TOL
    for b in (2, 4):     # the dense-layout kernel on the gathered sequence
        k_enc, v_enc = cache.fetch_sequence(bt[b], lens[b])
        one = tri.decode_step(t(q[b:b + 1], dev), SpectralEncoding(*(x[None] for x in k_enc)),
                              SpectralEncoding(*(x[None] for x in v_enc))).cpu().numpy()
        assert np.max(np.abs(one[0] - out[b])) <= 2e-6
    # float16 queries stay float16 inside the kernel (its own query table), bfloat16 ones are widened
    for qdt, npdt in ((torch.float16, np.float16),):
        qh = q.astype(npdt)
        out_h = tri.decode_step_paged(t(qh, dev), cache, bt, cl).cpu().numpy()
        ref_h = O.tri_decode_step_paged(qh.astype(np.float32), arrays, tables, lens, BS, tri._theta.cpu().numpy())
        assert np.max(np.abs(out_h - ref_h)) <= TOL
    qb = torch.from_numpy(q).to(dev).bfloat16()
    out_b = tri.decode_step_paged(qb, cache, bt, cl).cpu().numpy()
    ref_b = O.tri_decode_step_paged(qb.float().cpu().numpy(), arrays, tables, lens, BS, tri._theta.cpu().numpy())
    assert np.max(np.abs(out_b - ref_b)) <= TOL


def test_paged_decode_without_table_columns(dev):
    """A block table with no columns: every sequence is empty, the output is zero."""
    from aitherkvcache_amd.triattention import SpectralKVCache
    cfg = TriAttentionConfig(num_kv_heads=8, num_query_heads=32)
    tri = TriAttention(cfg, device=str(dev))
    cache = SpectralKVCache(cfg, max_blocks=4, device=str(dev))
    q = torch.randn(3, 32, 128, device=dev)
    out = tri.decode_step_paged(q, cache, torch.zeros(3, 0, dtype=torch.int32, device=dev),
                                torch.tensor([5, 0, 9], device=dev, dtype=torch.int32))
    assert out.shape == (3, 32, 128) and not bool(out.any())


@pytest.mark.parametrize("S", [1, 63, 64, 65, 200])
@pytest.mark.parametrize("qdtype", [torch.float32, torch.float16, torch.bfloat16])
def test_short_sequences_zero_and_large_values(dev, S, qdtype):
    """Sequences around one chunk of 64 tokens; value rows that are all zero (their stored scale is 0)
    and value rows a thousand times larger than the rest; float16 / bfloat16 queries."""
    cfg = TriAttentionConfig(num_kv_heads=8, num_query_heads=32)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(S)
    B, KVH, QH, D = 2, 8, 32, 128
    keys = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    vals = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    vals[:, ::3] = 0
    vals[:, 1::7] *= 1000
    k_enc, v_enc = tri.encode_kv(t(keys, dev), t(vals, dev))
    assert float(v_enc.scales[0, 0, 0]) == 0.0
    q = torch.from_numpy(rng.standard_normal((B, QH, D)).astype(np.float32)).to(dev).to(qdtype)
    out = tri.decode_step(q, k_enc, v_enc).cpu().numpy()
    ref = O.tri_decode_step(q.float().cpu().numpy(), tuple(x.cpu().numpy() for x in k_enc),
                            tuple(x.cpu().numpy() for x in v_enc), tri._theta.cpu().numpy())
    scale = max(1.0, float(np.abs(ref).max()))
    assert np.max(np.abs(out - ref)) <= TOL * scale


@pytest.mark.parametrize("qdtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kp_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("QH,KVH", [(32, 8), (16, 2), (6, 2)])
def test_key_positions_of_both_widths_and_query_types(dev, qdtype, kp_dtype, QH, KVH):
    """Explicit key positions (32- and 64-bit) with every query type on the all-heads kernel, over several
    ranges of a sequence; groups of four, eight (two groups on the grid) and three (one by one) query heads."""
    cfg = TriAttentionConfig(num_kv_heads=KVH, num_query_heads=QH)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(QH * 100 + KVH)
    B, S, D = 2, 1500, 128
    keys = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    vals = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    k_enc, v_enc = tri.encode_kv(t(keys, dev), t(vals, dev))
    q = torch.from_numpy(rng.standard_normal((B, QH, D)).astype(np.float32)).to(dev).to(qdtype)
    kpos = np.sort(rng.integers(0, 30000, size=(B, S)), axis=-1)
    qpos = np.array([31000, 40000])
    out = tri.decode_step(q, k_enc, v_enc, t(qpos, dev), torch.from_numpy(kpos).to(dev).to(kp_dtype)).cpu().numpy()
    ref = O.tri_decode_step(q.float().cpu().numpy(), tuple(x.cpu().numpy() for x in k_enc),
                            tuple(x.cpu().numpy() for x in v_enc), tri._theta.cpu().numpy(), qpos, kpos)
    assert np.max(np.abs(out - ref)) <= TOL * max(1.0, float(np.abs(ref).max()))


def test_scores_that_grow_along_the_sequence(dev):
    """Post-RoPE scoring of keys that are multiples of one vector, growing with the position: every chunk of 64
    tokens raises the running maxima (the sums are rescaled every time), and the last tokens carry the output."""
    cfg = TriAttentionConfig(num_kv_heads=8, num_query_heads=32, pre_rope=False)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(11)
    B, S, KVH, QH, D = 2, 2000, 8, 32, 128
    base = rng.standard_normal((1, 1, KVH, D))
    keys = (base * np.linspace(0.05, 3.0, S)[None, :, None, None]).astype(np.float16)
    vals = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    k_enc, v_enc = tri.encode_kv(t(np.broadcast_to(keys, (B, S, KVH, D)).copy(), dev), t(vals, dev))
    q = np.repeat(base[0, 0], QH // KVH, axis=0)[None].repeat(B, 0).astype(np.float32)      # aligned with the keys
    out = tri.decode_step(t(q, dev), k_enc, v_enc).cpu().numpy()
    ref = O.tri_decode_step(q, tuple(x.cpu().numpy() for x in k_enc), tuple(x.cpu().numpy() for x in v_enc),
                            tri._theta.cpu().numpy(), pre_rope=False)
    assert np.max(np.abs(out - ref)) <= TOL * max(1.0, float(np.abs(ref).max()))


def test_empty_batch_and_empty_sequence(dev):
    cfg = TriAttentionConfig(num_kv_heads=8, num_query_heads=32)
    tri = TriAttention(cfg, device=str(dev))

    def enc(b, s):
        return SpectralEncoding(torch.zeros(b, s, 8, 12, dtype=torch.uint8, device=dev),
                                torch.zeros(b, s, 8, 12, dtype=torch.uint8, device=dev),
                                torch.zeros(b, s, 8, dtype=torch.float16, device=dev))

    out = tri.decode_step(torch.randn(3, 32, 128, device=dev), enc(3, 0), enc(3, 0))
    assert out.shape == (3, 32, 128) and not bool(out.any())
    out0 = tri.decode_step(torch.randn(0, 32, 128, device=dev), enc(0, 5), enc(0, 5))
    assert out0.shape == (0, 32, 128)


# ---- coefficient widths 8 / 16 and post-RoPE scoring -------------------------------------------------
WIDTH_MODES = [(8, True), (16, True), (4, False), (8, False), (16, False)]


def _wenc(g, bits, nm, dev):
    return SpectralEncoding(*(t(g[f"enc_b{bits}_{nm}_{part}"], dev) for part in ("indices", "packed", "scales")))


@pytest.mark.parametrize("bits,pre", WIDTH_MODES)
def test_widths_and_post_rope_golden(golden, tri_widths, dev, bits, pre):
    """The reference's own encodings and outputs at coeff_bits 8 / 16 and with pre_rope=False: the
    write-side kernel reproduces the encodings bit for bit, decode_step the outputs to TOL."""
    g = tri_widths
    cfg = TriAttentionConfig(head_dim=128, num_freqs=12, coeff_bits=bits, num_kv_heads=2, num_query_heads=8,
                             rope_base=1_000_000.0, pre_rope=pre)
    tri = TriAttention(cfg, device=str(dev))
    k_enc, v_enc = tri.encode_kv(t(g["keys"], dev), t(g["vals"], dev))
    for nm, e in (("k", k_enc), ("v", v_enc)):
        for part, got in zip(("indices", "packed", "scales"), e):
            want = g[f"enc_b{bits}_{nm}_{part}"]
            assert got.cpu().numpy().dtype == want.dtype and got.shape == want.shape
            assert np.array_equal(got.cpu().numpy().view(np.uint8), want.view(np.uint8)), (nm, part)
    tag = f"b{bits}_{'pre' if pre else 'post'}"
    ke, ve = _wenc(g, bits, "k", dev), _wenc(g, bits, "v", dev)
    out = tri.decode_step(t(g["q"], dev), ke, ve, t(g["qpos"], dev), t(g["kpos"], dev)).cpu().numpy()
    e1 = np.max(np.abs(out - g[f"out_{tag}"]))
    out_d = tri.decode_step(t(g["q"], dev), ke, ve).cpu().numpy()
    e2 = np.max(np.abs(out_d - g[f"out_default_pos_{tag}"]))
    print(f"[tri widths golden] {tag}: explicit-pos {e1:.2e}, default-pos {e2:.2e}")
    assert e1 <= TOL and e2 <= TOL


@pytest.mark.parametrize("bits,pre", WIDTH_MODES)
@pytest.mark.parametrize("B,S,QH,KVH,D,F,base", [(2, 1000, 32, 8, 128, 12, 1e6), (2, 333, 6, 2, 32, 4, 1e4),
                                                 (1, 64, 4, 4, 64, 32, 1e4), (2, 700, 8, 2, 128, 20, 1e6),
                                                 (1, 3000, 16, 16, 128, 12, 1e6)])
def test_widths_and_post_rope_vs_oracle(dev, bits, pre, B, S, QH, KVH, D, F, base):
    cfg = TriAttentionConfig(head_dim=D, num_freqs=F, coeff_bits=bits, num_kv_heads=KVH, num_query_heads=QH,
                             rope_base=base, pre_rope=pre)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(S + bits)
    pair_std = (np.arange(D // 2) + 1.0) ** -0.75
    keys = (rng.standard_normal((B, S, KVH, D // 2, 2)) * pair_std[:, None]).reshape(B, S, KVH, D).astype(np.float16)
    vals = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    k_enc, v_enc = tri.encode_kv(t(keys, dev), t(vals, dev))
    ke, ve = O.spectral_encode(keys, F, bits), O.spectral_encode(vals, F, bits)
    for got, want in zip(tuple(k_enc) + tuple(v_enc), ke + ve):
        assert got.shape == want.shape and np.array_equal(got.cpu().numpy().view(np.uint8), want.view(np.uint8))
    q = rng.standard_normal((B, QH, D)).astype(np.float32)
    qpos = rng.integers(S, 40000, size=B)
    kpos = np.sort(rng.integers(0, 32768, size=(B, S)), axis=-1)
    theta = tri._theta.cpu().numpy()
    out = tri.decode_step(t(q, dev), k_enc, v_enc, t(qpos, dev), t(kpos, dev)).cpu().numpy()
    ref = O.tri_decode_step(q, ke, ve, theta, qpos, kpos, bits, pre)
    err = np.max(np.abs(out - ref))
    print(f"[tri widths] bits={bits} pre={pre} B={B} S={S} D={D} F={F} max|diff|={err:.2e} max|out|={np.abs(ref).max():.3f}")
    assert err <= TOL
    out_d = tri.decode_step(t(q, dev), k_enc, v_enc).cpu().numpy()
    ref_d = O.tri_decode_step(q, ke, ve, theta, None, None, bits, pre)
    assert np.max(np.abs(out_d - ref_d)) <= TOL
    if not pre:                      # positions play no part
        assert np.array_equal(out, out_d)


@pytest.mark.parametrize("bits", [8, 16])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_spectral_encode_widths_vs_oracle(dev, bits, dtype):
    D, F = 128, 12
    rng = np.random.default_rng(bits)
    n = 5000
    x = (rng.standard_normal((n, D)) * rng.lognormal(0, 1.0, (n, 1))).astype(np.float32)
    x[7] = 0.0
    x[8, 2:] = 0.0
    x[9] *= 1e-6
    xt = torch.from_numpy(x).to(dev).to(dtype)
    tri = TriAttention(TriAttentionConfig(head_dim=D, num_freqs=F, coeff_bits=bits, num_kv_heads=1, num_query_heads=1),
                       device=str(dev))
    e = tri.encoder.encode(xt)
    ri, rp, rs = O.spectral_encode(xt.float().cpu().numpy(), F, bits)
    assert np.array_equal(e.indices.cpu().numpy(), ri)
    assert e.packed.shape == rp.shape and np.array_equal(e.packed.cpu().numpy().view(np.uint8), rp.view(np.uint8))
    assert np.array_equal(e.scales.cpu().numpy(), rs)
    # the host path (torch ops) of the encoder and the dense reconstruction agree with the kernel's encoding
    # (rows without pairs of equal energy: torch.topk leaves the order among ties open)
    eh = tri.encoder.encode(xt[10:].cpu())
    assert torch.equal(eh.indices, e.indices[10:].cpu()) and torch.equal(eh.packed, e.packed[10:].cpu())
    assert torch.equal(eh.scales, e.scales[10:].cpu())
    dec = tri.encoder.decode(e).cpu().numpy()
    v0, v1 = O.unpack_coefficients(rp, rs, bits)
    want = np.zeros((n, D), np.float32)
    np.put_along_axis(want, 2 * ri.astype(np.int64), v0, -1)
    np.put_along_axis(want, 2 * ri.astype(np.int64) + 1, v1, -1)
    # torch's device division may differ in the last place of code / half (values near 1): an absolute
    # 2^-22 of the row's scale
    assert np.all(np.abs(dec - want) <= 2.5e-7 * rs.astype(np.float32)[:, None])
    e0 = tri.encoder.encode(xt[:0])
    assert e0.indices.shape == (0, F) and e0.packed.shape[0] == 0


def test_paged_decode_post_rope_vs_oracle(dev):
    """The paged kernel with pre_rope=False: block pool of int4 rows, ragged contexts, against the oracle's
    fetch_sequence + decode_step per sequence."""
    from aitherkvcache_amd.triattention import SpectralKVCache
    KVH, QH, BS = 8, 32, 16
    cfg = TriAttentionConfig(head_dim=128, num_freqs=12, num_kv_heads=KVH, num_query_heads=QH, block_size=BS,
                             pre_rope=False)
    tri = TriAttention(cfg, device=str(dev))
    cache = SpectralKVCache(cfg, max_blocks=64, device=str(dev))
    rng = np.random.default_rng(77)
    ctx = np.array([200, 0, 33, 512], dtype=np.int64)
    B, MB = len(ctx), 32
    perm = rng.permutation(64)
    bt = np.zeros((B, MB), dtype=np.int32)
    used = 0
    for b in range(B):
        nb = -(-int(ctx[b]) // BS)
        bt[b, :nb] = perm[used:used + nb]          # 13 + 0 + 3 + 32 blocks of the 64
        used += nb
    keys = rng.standard_normal((64 * BS, KVH, 128)).astype(np.float16)
    vals = rng.standard_normal((64 * BS, KVH, 128)).astype(np.float16)
    ke = tri.encoder.encode(t(keys, dev))
    ve = tri.encoder.encode(t(vals, dev))
    for dst, src in zip(cache._arrays(), tuple(ke) + tuple(ve)):
        dst.copy_(src.reshape(dst.shape))
    q = rng.standard_normal((B, QH, 128)).astype(np.float32)
    out = tri.decode_step_paged(t(q, dev), cache, t(bt, dev), t(ctx, dev)).cpu().numpy()
    arrays = tuple(a.cpu().numpy() for a in cache._arrays())
    ref = O.tri_decode_step_paged(q, arrays, bt, ctx, BS, tri._theta.cpu().numpy(), None, 4, False)
    err = np.max(np.abs(out - ref))
    print(f"[tri paged post-rope] max|diff|={err:.2e}")
    assert err <= TOL and np.all(out[1] == 0)
    # and it differs from the pre-RoPE result (the flag is not ignored)
    tri_pre = TriAttention(TriAttentionConfig(head_dim=128, num_freqs=12, num_kv_heads=KVH, num_query_heads=QH,
                                              block_size=BS), device=str(dev))
    out_pre = tri_pre.decode_step_paged(t(q, dev), cache, t(bt, dev), t(ctx, dev)).cpu().numpy()
    assert np.max(np.abs(out_pre - out)) > 1e-3


def test_width_argument_checks(dev):
    cfg = TriAttentionConfig(head_dim=128, num_freqs=12, coeff_bits=8, num_kv_heads=2, num_query_heads=8)
    tri = TriAttention(cfg, device=str(dev))
    x = torch.randn(1, 10, 2, 128, device=dev).half()
    k_enc, v_enc = tri.encode_kv(x, x)
    assert k_enc.packed.shape == (1, 10, 2, 24)
    tri4 = TriAttention(TriAttentionConfig(head_dim=128, num_freqs=12, num_kv_heads=2, num_query_heads=8), device=str(dev))
    with pytest.raises(ValueError):          # 8-bit rows handed to a 4-bit configuration
        tri4.decode_step(torch.randn(1, 8, 128, device=dev), k_enc, v_enc)
    from aitherkvcache_amd import _lib
    L = _lib.lib()
    rc = L.akv_tri_encode(x.data_ptr(), _lib.dtype_code(x), 20, 128, 128, 12, 5, x.data_ptr(), x.data_ptr(), x.data_ptr(), None)
    assert rc == _lib.AKV_ERR_INVALID


# ---- the scorer alone, the prefill form, helpers ------------------------------------------------------
def test_scorer_golden(golden, tri_widths, dev):
    """TrigSeriesScorer.score against the reference's own logits: default width with explicit positions, and the
    other widths / post-RoPE."""
    from aitherkvcache_amd.triattention import TrigSeriesScorer
    cfg = TriAttentionConfig(head_dim=128, num_freqs=12, coeff_bits=4, num_kv_heads=2, num_query_heads=8, rope_base=1e6)
    sc = TrigSeriesScorer(cfg, device=str(dev)).score(t(golden["tri_q"], dev), enc(golden, "k", dev),
                                                      t(golden["tri_qpos"], dev), t(golden["tri_kpos"], dev))
    assert sc.dtype == torch.float32 and sc.shape == golden["tri_scores_explicit_pos"].shape
    e = np.max(np.abs(sc.cpu().numpy() - golden["tri_scores_explicit_pos"]))
    print(f"[tri scorer golden] {e:.2e}")
    assert e <= TOL
    g = tri_widths
    for bits, pre in WIDTH_MODES:
        cfg = TriAttentionConfig(head_dim=128, num_freqs=12, coeff_bits=bits, num_kv_heads=2, num_query_heads=8,
                                 rope_base=1e6, pre_rope=pre)
        got = TrigSeriesScorer(cfg, device=str(dev)).score(t(g["q"], dev), _wenc(g, bits, "k", dev), t(g["qpos"], dev),
                                                           t(g["kpos"], dev)).cpu().numpy()
        assert np.max(np.abs(got - g[f"scores_b{bits}_{'pre' if pre else 'post'}"])) <= TOL


@pytest.mark.parametrize("B,S,QH,KVH,D,F,bits", [(2, 700, 32, 8, 128, 12, 4), (2, 333, 6, 2, 32, 4, 8), (1, 70, 4, 4, 64, 32, 16)])
def test_scorer_vs_oracle(dev, B, S, QH, KVH, D, F, bits):
    cfg = TriAttentionConfig(head_dim=D, num_freqs=F, coeff_bits=bits, num_kv_heads=KVH, num_query_heads=QH, rope_base=1e4)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(S)
    keys = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    k_enc, _ = tri.encode_kv(t(keys, dev), t(keys, dev))
    q = rng.standard_normal((B, QH, D)).astype(np.float32)
    qpos = rng.integers(S, 9000, size=B)
    kpos = np.sort(rng.integers(0, 8000, size=(B, S)), axis=-1)
    theta = tri._theta.cpu().numpy()
    ke = tuple(x.cpu().numpy() for x in k_enc)
    got = tri.scorer.score(t(q, dev), k_enc, t(qpos, dev), t(kpos, dev)).cpu().numpy()
    assert np.max(np.abs(got - O.tri_scores(q, *ke, theta, qpos, kpos, bits))) <= TOL
    got = tri.scorer.score(t(q, dev), k_enc).cpu().numpy()              # default positions
    assert np.max(np.abs(got - O.tri_scores(q, *ke, theta, None, None, bits))) <= TOL
    one = tri.scorer.score_single(t(q[:1], dev), SpectralEncoding(*(x[:1] for x in k_enc)), 1234).cpu().numpy()
    assert np.max(np.abs(one - O.tri_scores(q[:1], *(x[:1] for x in ke), theta, np.array([1234]), None, bits))) <= TOL


@pytest.mark.parametrize("masked", [False, True])
def test_forward_prefill_form_vs_oracle(dev, masked):
    """TriAttention.forward: encode, then every query position i at position i against all keys, with and without an
    additive (causal) mask; single-query form squeezed."""
    B, S, Sq, QH, KVH, D, F = 2, 90, 5, 8, 2, 128, 12
    cfg = TriAttentionConfig(head_dim=D, num_freqs=F, num_kv_heads=KVH, num_query_heads=QH, rope_base=1e4)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(5)
    keys = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    vals = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
    q = rng.standard_normal((B, QH, Sq, D)).astype(np.float32)
    mask = None
    if masked:
        mask = np.zeros((B, Sq, S), np.float32)
        for i in range(Sq):
            mask[:, i, 40 + 10 * i:] = -np.inf
    out = tri.forward(t(q, dev), t(keys, dev), t(vals, dev), attention_mask=None if mask is None else t(mask, dev))
    assert out.shape == (B, QH, Sq, D) and out.dtype == torch.float32
    ke, ve = O.spectral_encode(keys, F), O.spectral_encode(vals, F)
    theta = tri._theta.cpu().numpy()
    for i in range(Sq):
        ref = O.tri_decode_step(q[:, :, i], ke, ve, theta, np.full((B,), i), None, 4, True,
                                None if mask is None else mask[:, i:i + 1])
        assert np.max(np.abs(out[:, :, i].cpu().numpy() - ref)) <= TOL
    one = tri.forward(t(q[:, :, 0], dev), t(keys, dev), t(vals, dev))
    assert one.shape == (B, QH, D) and torch.equal(one, tri.forward(t(q[:, :, :1], dev), t(keys, dev), t(vals, dev))[:, :, 0])


def test_full_series_equals_rope_attention(dev):
    """All pairs kept as fp16: the trigonometric series is RoPE attention (reference test_triattention.py:183-208)."""
    B, S, QH, KVH, D = 2, 50, 4, 2, 32
    cfg = TriAttentionConfig(head_dim=D, num_freqs=D // 2, coeff_bits=16, num_kv_heads=KVH, num_query_heads=QH, rope_base=1e4)
    tri = TriAttention(cfg, device=str(dev))
    g = torch.Generator(device=dev).manual_seed(1)
    q = torch.randn(B, QH, D, device=dev, generator=g)
    k = torch.randn(B, S, KVH, D, device=dev, generator=g).half()
    v = torch.randn(B, S, KVH, D, device=dev, generator=g).half()
    qpos = torch.tensor([60, 75], device=dev)
    kpos = torch.arange(S, device=dev).unsqueeze(0).expand(B, -1)
    out = tri.decode_step(q, *tri.encode_kv(k, v), qpos, kpos)
    ref = TriAttention.reference_attention(q, k, v, 1e4, qpos, kpos)
    assert torch.max(torch.abs(out - ref)).item() < 1e-3
    stats = tri.encoder.compression_stats(k)
    assert stats["cosine_similarity"] > 0.999 and stats["energy_ratio"] > 0.999


@pytest.mark.gpu
def test_benchmark_method_reports_times_and_quality(dev):
    """TriAttention.benchmark runs encode, decode step and the dense reference on random data; random vectors have
    no spectral concentration, so only the shape of the report and sane ranges are asserted."""
    from aitherkvcache_amd.triattention import TriAttention, TriAttentionConfig
    tri = TriAttention(TriAttentionConfig(head_dim=128, num_freqs=12, num_kv_heads=2, num_query_heads=8), device=str(dev))
    rep = tri.benchmark(batch_size=2, seq_len=300, num_trials=2)
    assert set(rep) == {"encode_ms", "decode_ms", "reference_ms", "speedup", "compression_ratio", "cosine_similarity",
                        "mse", "seq_len", "batch_size"}
    assert rep["encode_ms"] > 0 and rep["decode_ms"] > 0 and rep["reference_ms"] > 0
    assert rep["seq_len"] == 300 and rep["batch_size"] == 2 and rep["compression_ratio"] > 5
    assert -1.0 <= rep["cosine_similarity"] <= 1.0 and rep["mse"] >= 0


@pytest.mark.parametrize("KVH,BS,dtype,it", [(8, 16, torch.float16, torch.int64), (2, 8, torch.bfloat16, torch.int32),
                                             (4, 24, torch.float32, torch.int64)])
def test_encode_on_write_into_the_paged_cache(dev, KVH, BS, dtype, it):
    """SpectralKVCache.encode_and_store: a step's keys and values encoded and written into the block pool by one
    launch per tensor -- the rows are those of encode (byte for byte, and the oracle's), they land at their slots,
    skipped tokens (negative slots, slots past the cache) and every other row stay untouched; strided inputs; a
    decode step over the written cache agrees with the oracle."""
    from aitherkvcache_amd.triattention import SpectralKVCache
    cfg = TriAttentionConfig(num_kv_heads=KVH, num_query_heads=4 * KVH, block_size=BS)
    tri = TriAttention(cfg, device=str(dev))
    rng = np.random.default_rng(300 + KVH)
    NB, T, D = 12, 70, 128
    cache = SpectralKVCache(cfg, max_blocks=NB, device=str(dev))
    for a in cache._arrays():
        a.fill_(7)
    pair_std = (np.arange(D // 2) + 1.0) ** -0.75
    keys = (rng.standard_normal((T, KVH, D // 2, 2)) * pair_std[:, None]).reshape(T, KVH, D).astype(np.float32)
    vals = rng.standard_normal((T, KVH, D)).astype(np.float32)
    kd, vd = t(keys, dev).to(dtype), t(vals, dev).to(dtype)
    wide = torch.zeros(T, KVH, D + 8, dtype=dtype, device=dev)       # values through a strided view
    wide[..., :D] = vd
    slots = rng.permutation(NB * BS)[:T].astype(np.int64)
    slots[::11] = -1
    slots[5] = NB * BS + 3
    cache.encode_and_store(kd, wide[..., :D], t(slots, dev).to(it))
    k_enc, v_enc = tri.encode_kv(kd[None], vd[None])
    ok = (slots >= 0) & (slots < NB * BS)
    arrays = [a.cpu().numpy() for a in cache._arrays()]
    for got, want in zip(arrays, [x[0].cpu().numpy() for x in tuple(k_enc) + tuple(v_enc)]):
        flat = got.reshape((NB * BS,) + got.shape[2:])
        assert np.array_equal(flat[slots[ok]], want[ok])
        untouched = np.ones(NB * BS, bool)
        untouched[slots[ok]] = False
        assert np.all(flat[untouched] == 7)
    ref = O.spectral_encode(kd.float().cpu().numpy(), 12, 4)
    assert np.array_equal(arrays[0].reshape(NB * BS, KVH, 12)[slots[ok]], ref[0][ok])
    assert np.array_equal(arrays[1].reshape(NB * BS, KVH, 12)[slots[ok]], ref[1][ok])
    # the written tokens as one sequence, read back through a block table
    seq = np.flatnonzero(ok)[:BS * 3]
    cache2 = SpectralKVCache(cfg, max_blocks=NB, device=str(dev))
    table = rng.permutation(NB)[:4]
    sl = np.array([table[j // BS] * BS + j % BS for j in range(len(seq))], dtype=np.int64)
    cache2.encode_and_store(kd[seq], vd[seq], torch.from_numpy(sl))               # (slots as host data)
    q = rng.standard_normal((1, 4 * KVH, D)).astype(np.float32)
    out = tri.decode_step_paged(t(q, dev), cache2, t(table[None], dev), torch.tensor([len(seq)], device=dev)).cpu().numpy()
    refo = O.tri_decode_step_paged(q, [a.cpu().numpy() for a in cache2._arrays()], table[None], [len(seq)], BS,
                                   tri._theta.cpu().numpy())
    assert np.max(np.abs(out - refo)) <= TOL
    assert cache2.memory_stats()["used_blocks"] == -(-len(seq) // BS)

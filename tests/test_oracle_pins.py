"""Checks that pin the oracle by means other than the golden file: exhaustive brute force on
the bit layouts, the library routine the quantiser reduces to, closed forms and identities the
reference's own tests use (tests/test_core.py, test_fused.py, test_triattention.py)."""
import itertools
import math

import numpy as np
import pytest

from oracle import tq_oracle as O


# ---- packing: documented layouts, brute force ------------------------------------------
def test_pack4_every_byte():
    idx = np.array(list(itertools.product(range(16), repeat=2)), dtype=np.uint8)   # all 256 pairs
    p = O.pack_4bit(idx)
    assert np.array_equal(p[:, 0], idx[:, 0] * 16 + idx[:, 1])
    assert np.array_equal(O.unpack_4bit(p, 2), idx)
    assert sorted(p[:, 0].tolist()) == list(range(256))


def test_pack2_every_byte():
    idx = np.array(list(itertools.product(range(4), repeat=4)), dtype=np.uint8)
    p = O.pack_2bit(idx)
    assert np.array_equal(p[:, 0], idx[:, 0] * 64 + idx[:, 1] * 16 + idx[:, 2] * 4 + idx[:, 3])
    assert np.array_equal(O.unpack_2bit(p, 4), idx)
    assert sorted(p[:, 0].tolist()) == list(range(256))


def test_pack3_every_24bit_word():
    # all 2**24 words: value i sits at bits 23-3i..21-3i of the big-endian 3-byte word
    w = np.arange(1 << 24, dtype=np.int64)
    idx = np.stack([(w >> (21 - 3 * i)) & 7 for i in range(8)], axis=1).astype(np.uint8)
    p = O.pack_3bit(idx)
    word = (p[:, 0].astype(np.int64) << 16) | (p[:, 1].astype(np.int64) << 8) | p[:, 2]
    assert np.array_equal(word, w)
    assert np.array_equal(O.unpack_3bit(p, 8), idx)


@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_multibit_is_msb_first_stream(bits):
    rng = np.random.default_rng(bits)
    idx = rng.integers(0, 1 << bits, size=(50, 64))
    p = O.pack_multibit(idx, bits)
    assert p.shape == (50, math.ceil(64 * bits / 8))
    # independent statement: write the indices as a binary string, cut it into bytes
    for r in range(50):
        s = "".join(format(int(v), f"0{bits}b") for v in idx[r])
        expect = [int(s[i:i + 8].ljust(8, "0"), 2) for i in range(0, len(s), 8)]
        assert p[r].tolist() == expect
    assert np.array_equal(O.unpack_multibit(p, 64, bits), idx)
    # the fixed-width packers are the same stream
    fixed = {2: O.pack_2bit, 3: O.pack_3bit, 4: O.pack_4bit}
    if bits in fixed:
        assert np.array_equal(fixed[bits](idx), p)


def test_packed_sizes():
    assert [O.packed_size(128, b) for b in (4, 3, 2)] == [64, 48, 32]
    with pytest.raises(ValueError):
        O.packed_size(128, 5)


# ---- codebooks -----------------------------------------------------------------------
@pytest.mark.parametrize("bits", [2, 3, 4])
def test_codebook_structure(bits):
    c, b, mse = O.get_codebook(128, bits)
    assert len(c) == 1 << bits and len(b) == (1 << bits) - 1
    assert np.all(np.diff(c) > 0) and np.allclose(c, -c[::-1])
    assert np.allclose(b, (c[:-1].astype(np.float64) + c[1:]) / 2, atol=1e-9)
    c1, _, _ = O.get_codebook(1, bits)
    assert np.allclose(c * math.sqrt(128), c1, rtol=1e-6)          # 1/sqrt(d) scaling
    lo, hi = O.theory_bounds(bits)
    assert lo <= mse <= hi
    # Lloyd-Max fixed point for N(0,1): each level is the conditional mean of its cell
    from scipy import integrate, stats
    edges = np.concatenate([[-np.inf], (c1[:-1].astype(np.float64) + c1[1:]) / 2, [np.inf]])
    for k in range(len(c1)):
        num = integrate.quad(lambda x: x * stats.norm.pdf(x), edges[k], edges[k + 1])[0]
        den = stats.norm.cdf(edges[k + 1]) - stats.norm.cdf(edges[k])
        assert abs(num / den - c1[k]) < 1e-3      # tables carry 6 decimals


# ---- quantise: searchsorted(right=False) == brute-force count of boundaries below ------
@pytest.mark.parametrize("bits", [2, 3, 4])
def test_quantize_is_count_of_boundaries_below(bits):
    _, b, _ = O.get_codebook(128, bits)
    rng = np.random.default_rng(0)
    y = np.concatenate([rng.normal(0, 0.09, 5000).astype(np.float32), b, np.nextafter(b, np.inf),
                        np.nextafter(b, -np.inf), [0.0, -0.0, 10.0, -10.0]]).astype(np.float32)
    brute = np.array([sum(1 for t in b if t < v) for v in y])
    assert np.array_equal(O.quantize(y, b, bits), brute)
    # a value equal to a boundary belongs to the lower bin
    assert np.array_equal(O.quantize(b, b, bits), np.arange(len(b)))


# ---- encode / decode quality (reference tests/test_core.py:246-365) -------------------
@pytest.mark.parametrize("bits,table_mse", [(4, 0.0095), (3, 0.0345), (2, 0.1175)])
def test_round_trip_distortion(golden, bits, table_mse):
    R = golden["rotation_d128_seed42"]
    c, b, _ = O.get_codebook(128, bits)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((20000, 128)).astype(np.float32)
    x /= np.linalg.norm(x, axis=-1, keepdims=True)
    p, n = O.encode(x, R, b, bits)
    assert np.allclose(n, 1.0, atol=1e-5)
    xh = O.decode(p, n, R, c, bits, out_dtype=np.float32)
    mse = float(np.mean(np.sum((x - xh) ** 2, axis=-1)))
    lo, hi = O.theory_bounds(bits)
    assert lo <= mse <= hi
    assert abs(mse - table_mse) / table_mse < 0.05


def test_rotation_fixture_is_orthogonal(golden):
    for key in ("rotation_d128_seed42", "rotation_d64_seed42", "rotation_d128_seed7"):
        R = golden[key].astype(np.float64)
        assert np.allclose(R @ R.T, np.eye(R.shape[0]), atol=2e-6)
    assert not np.allclose(golden["rotation_d128_seed42"], golden["rotation_d128_seed7"])


def test_zero_vector_round_trip(golden):
    R = golden["rotation_d128_seed42"]
    c, b, _ = O.get_codebook(128, 4)
    p, n = O.encode(np.zeros((1, 128), np.float16), R, b, 4)
    assert n[0] == 0 and np.all(p == 0x77)
    assert np.all(O.decode(p, n, R, c, 4) == 0)


# ---- attention: the rotated-domain form equals decompress + dense attention ----------
@pytest.mark.parametrize("bits", [2, 3, 4])
def test_paged_attention_equals_decompress_then_dense(golden, bits):
    R = golden["rotation_d128_seed42"]
    c, b, _ = O.get_codebook(128, bits)
    rng = np.random.default_rng(7)
    NB, BS, KVH, QH = 9, 16, 2, 4
    keys = rng.standard_normal((NB * BS, KVH, 128)).astype(np.float16)
    vals = rng.standard_normal((NB * BS, KVH, 128)).astype(np.float16)
    kp, kn = O.encode(keys, R, b, bits)
    vp, vn = O.encode(vals, R, b, bits)
    P = kp.shape[-1]
    kp, vp = kp.reshape(NB, BS, KVH, P), vp.reshape(NB, BS, KVH, P)
    kn, vn = kn.reshape(NB, BS, KVH), vn.reshape(NB, BS, KVH)
    ctx = np.array([33, 0, 16, 5])
    tables = np.array([[4, 2, 7], [0, 0, 0], [8, 0, 0], [1, 0, 0]])
    q = rng.standard_normal((4, QH, 128)).astype(np.float32)
    fused = O.paged_attention(q, kp, kn, vp, vn, tables, ctx, R, c, bits, dtype=np.float64, cast_output=False)
    loop = O.paged_attention_loop(q, kp, kn, vp, vn, tables, ctx, R, c, bits)
    assert np.max(np.abs(loop - fused)) < 1e-5
    # brute force: decode every addressed token to the original domain, ordinary attention
    for s in range(4):
        if ctx[s] == 0:
            assert np.all(fused[s] == 0)
            continue
        slots = [tables[s, t // BS] * BS + t % BS for t in range(ctx[s])]
        kd = O.decode(kp.reshape(-1, KVH, P)[slots], kn.reshape(-1, KVH)[slots], R, c, bits, np.float64)
        vd = O.decode(vp.reshape(-1, KVH, P)[slots], vn.reshape(-1, KVH)[slots], R, c, bits, np.float64)
        dense = O.dense_attention(q[s], kd, vd, 1 / math.sqrt(128), dtype=np.float64)
        assert np.max(np.abs(dense - fused[s])) < 2e-5
    # permuting physical blocks together with the table changes nothing
    perm = rng.permutation(NB)
    inv = np.argsort(perm)
    fused2 = O.paged_attention(q, kp[perm], kn[perm], vp[perm], vn[perm], inv[tables], ctx, R, c, bits,
                               dtype=np.float64, cast_output=False)
    assert np.max(np.abs(fused2 - fused)) < 1e-12


# ---- hybrid ------------------------------------------------------------------------------
def test_batch_decompress_touches_exactly_the_listed_blocks(golden):
    # per-block loop: a listed block inside the cache equals decode() of that block alone, every
    # other block of the buffer keeps its sentinel; duplicates, negatives and ids past the cache
    rng = np.random.default_rng(5)
    R = golden["rotation_d128_seed42"]
    c, b, _ = O.get_codebook(128, 4)
    B, bs, H = 12, 4, 2
    x = rng.standard_normal((B, bs, H, 128)).astype(np.float32)
    packed, norms = O.encode(x, R, b, 4)
    cache = np.concatenate([packed, rng.integers(0, 256, (B, bs, H, 8), dtype=np.uint8)], axis=-1)
    table = np.array([[3, 7, -1, -1], [7, 0, 11, 10], [9, 40, -1, -1]])
    num_blocks = 10                                     # 10, 11 and 40 are outside the cache
    buf = np.full((B, bs, H, 128), 77, dtype=np.float16)
    O.batch_decompress_active_blocks(cache, norms, buf, table, num_blocks, R, c, 4, 64)
    for blk in range(B):
        if blk in (0, 3, 7, 9):
            one = O.decode(packed[blk], norms[blk], R, c, 4).astype(np.float32)   # BLAS sums in another order
            assert np.max(np.abs(buf[blk].astype(np.float32) - one)) <= 2e-3
        else:
            assert np.all(buf[blk] == 77)


def test_fwht_is_the_hadamard_matrix():
    H = np.array([[1.0]])
    while H.shape[0] < 64:
        H = np.block([[H, H], [H, -H]])
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 64)).astype(np.float32)
    assert np.allclose(O.fwht(x), x @ H.T, atol=1e-4)
    s = np.sign(rng.standard_normal(64)).astype(np.float32)
    y = O.structured_hadamard(x, s)
    assert np.allclose(y, (x * s) @ H.T / 8, atol=1e-5)
    assert np.allclose(O.structured_hadamard(y, s, inverse=True), x, atol=1e-5)      # unitary
    assert np.allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)


def test_hybrid_layout_and_quality(golden):
    hp = O.HybridParams(golden["hyb_g0_had_signs"], golden["hyb_g1_had_signs"],
                        golden["hyb_g0_qjl_signs"], golden["hyb_g1_qjl_signs"])
    assert hp.group_bytes == (36, 28) and hp.packed_dim == 64
    rng = np.random.default_rng(5)
    x = rng.standard_normal((4000, 128)).astype(np.float32)
    x /= np.linalg.norm(x, axis=-1, keepdims=True)
    p = O.hybrid_encode(x, hp)
    assert p.shape == (4000, 64) and p.dtype == np.uint8
    # norms are stored little-endian fp16 at bytes 32..33 and 60..61
    n0 = np.ascontiguousarray(p[:, 32:34]).view("<f2").reshape(-1).astype(np.float32)
    assert np.allclose(n0, np.linalg.norm(x[:, :64], axis=-1), rtol=1e-3)
    xh = O.hybrid_decode(p, hp)
    mse = float(np.mean(np.sum((x - xh) ** 2, axis=-1)))
    # 3-bit MSE on one half and 2-bit MSE on the other give (0.0345 + 0.1175) / 2 = 0.076 for a
    # unit vector before the QJL term; the sketch must bring it below that.  (The reference's
    # README quotes 0.0130 for tq35, README.md:472-480; its code -- which this oracle reproduces
    # bit for bit on the golden vectors -- does not reach that figure.)
    assert 0.03 < mse < 0.070
    cos = np.sum(x * xh, axis=-1) / np.linalg.norm(xh, axis=-1)
    assert cos.mean() > 0.95      # reference bar: > 0.7 (tests/test_hybrid_hooks.py:111-118)
    # decode of a batch equals decode of its slices
    assert np.array_equal(O.hybrid_decode(p[:7], hp), xh[:7])
    # dropping the QJL term must make the reconstruction worse (sign / scale of the sketch)
    p0 = p.copy()
    p0[:, 34:36] = 0
    p0[:, 62:64] = 0
    assert np.mean(np.sum((x - O.hybrid_decode(p0, hp)) ** 2, axis=-1)) > mse * 1.2


def test_hybrid_attention_is_attention_over_decoded_rows(golden):
    hp = O.HybridParams(golden["hyb_g0_had_signs"], golden["hyb_g1_had_signs"],
                        golden["hyb_g0_qjl_signs"], golden["hyb_g1_qjl_signs"])
    rng = np.random.default_rng(8)
    NB, BS, KVH, QH = 5, 16, 2, 4
    kc = O.hybrid_encode(rng.standard_normal((NB, BS, KVH, 128)).astype(np.float16), hp)
    vc = O.hybrid_encode(rng.standard_normal((NB, BS, KVH, 128)).astype(np.float16), hp)
    q = rng.standard_normal((2, QH, 128)).astype(np.float32)
    out = O.hybrid_paged_attention(q, kc, vc, np.array([[3, 1], [0, 0]]), np.array([20, 0]), hp, 0.1)
    assert np.all(out[1] == 0)
    kd = O.hybrid_decode(np.concatenate([kc[3], kc[1]])[:20], hp)
    vd = O.hybrid_decode(np.concatenate([vc[3], vc[1]])[:20], hp)
    for qh in range(QH):
        s = (kd[:, qh // 2] @ q[0, qh]) * 0.1
        w = np.exp(s - s.max())
        w /= w.sum()
        assert np.allclose(out[0, qh], w @ vd[:, qh // 2], atol=1e-5)


# ---- TriAttention: trig series == explicit RoPE attention (reference test_triattention.py:183-208) --
def _apply_rope(x, pos, theta):
    ang = pos[..., None] * theta
    c, s = np.cos(ang), np.sin(ang)
    out = np.empty_like(x)
    out[..., 0::2] = x[..., 0::2] * c - x[..., 1::2] * s
    out[..., 1::2] = x[..., 0::2] * s + x[..., 1::2] * c
    return out


def test_tri_full_series_equals_rope_attention():
    D, S, B, KVH, QH = 32, 24, 2, 2, 4
    rng = np.random.default_rng(11)
    theta = O.rope_frequencies(D, 10000.0).astype(np.float64)
    keys = rng.standard_normal((B, S, KVH, D))
    q = rng.standard_normal((B, QH, D))
    # encode with every pair kept; make the int4 grid exact by choosing values on it
    levels = (np.arange(16) / 7.5 - 1.0)
    keys = levels[rng.integers(0, 16, size=keys.shape)] * 2.0
    keys[..., 0] = 2.0                                     # pins the per-token scale at 2.0
    idx, packed, scales = O.spectral_encode(keys.astype(np.float32), D // 2)
    assert np.all(scales == 2.0)
    k0, k1 = O.unpack_coefficients(packed, scales)
    assert np.allclose(k0, keys[..., 0::2], atol=1e-6) and np.allclose(k1, keys[..., 1::2], atol=1e-6)
    qpos = np.array([40, 7])
    kpos = np.stack([np.arange(S), np.arange(S) * 2 + 1])
    sc = O.tri_scores(q.astype(np.float32), idx, packed, scales, theta.astype(np.float32), qpos, kpos)
    q_r = _apply_rope(q, qpos[:, None].astype(np.float64), theta)
    k_r = _apply_rope(keys, kpos[:, :, None].astype(np.float64), theta)
    for b in range(B):
        for h in range(QH):
            exact = k_r[b, :, h // 2] @ q_r[b, h] / math.sqrt(D)
            assert np.max(np.abs(sc[b, h] - exact)) < 1e-3
    # decode_step = softmax(scores) applied to the dequantised values
    vals = levels[rng.integers(0, 16, size=keys.shape)]
    vals[..., 0] = 1.0
    ve = O.spectral_encode(vals.astype(np.float32), D // 2)
    out = O.tri_decode_step(q.astype(np.float32), (idx, packed, scales), ve, theta.astype(np.float32), qpos, kpos)
    for b in range(B):
        for h in range(QH):
            w = np.exp(sc[b, h] - sc[b, h].max())
            w /= w.sum()
            assert np.allclose(out[b, h], w @ vals[b, :, h // 2], atol=1e-5)


def test_tri_truncation_keeps_largest_pairs():
    rng = np.random.default_rng(12)
    x = rng.standard_normal((50, 128)).astype(np.float32)
    idx, packed, scales = O.spectral_encode(x, 12)
    en = (x.reshape(50, 64, 2) ** 2).sum(-1)
    assert np.all(np.diff(idx.astype(int), axis=-1) > 0)          # ascending, distinct
    for r in range(50):
        assert set(idx[r].tolist()) == set(np.argsort(-en[r])[:12].tolist())
    assert idx.shape[-1] + packed.shape[-1] + 2 == 26             # bytes per token


def test_spectral_fetch_sequence_is_token_by_token_indexing():
    """fetch_sequence (reference: triattention/cache.py:163-198) against a loop that looks every token up
    by (block_table[t // block_size], t % block_size); permuted tables, a ragged last block, padding entries."""
    rng = np.random.default_rng(11)
    NB, BS, KVH, F = 9, 4, 2, 3
    arrays = [rng.integers(0, 256, size=(NB, BS, KVH, F), dtype=np.uint8) for _ in range(2)]
    arrays.append(rng.standard_normal((NB, BS, KVH)).astype(np.float16))
    arrays += [rng.integers(0, 256, size=(NB, BS, KVH, F), dtype=np.uint8) for _ in range(2)]
    arrays.append(rng.standard_normal((NB, BS, KVH)).astype(np.float16))
    table = np.array([7, 2, 5, 0, 99, -1])          # the last two are padding: never dereferenced
    for n in (1, 4, 5, 15, 16):
        k_enc, v_enc = O.spectral_fetch_sequence(arrays, table, n, BS)
        for j, got in enumerate(k_enc + v_enc):
            want = np.stack([arrays[j][table[t // BS], t % BS] for t in range(n)])
            assert got.shape == want.shape and np.array_equal(got, want)


def test_hybrid_margins_accept_the_oracle_and_catch_defects(golden):
    """hybrid_encode_margins (float64) against the float32 oracle: no code or sign of the oracle's own
    rows, nor of the reference's golden rows, is more than a rounding away from the float64 answer, and
    a flipped code bit or sign bit shows up as a margin of millions of ulps."""
    books = tuple((golden[f"hyb_centroids_64_{k}"], golden[f"hyb_boundaries_64_{k}"]) for k in (3, 2))
    hp = O.HybridParams(golden["hyb_g0_had_signs"], golden["hyb_g1_had_signs"],
                        golden["hyb_g0_qjl_signs"], golden["hyb_g1_qjl_signs"], codebooks=books)
    m = O.hybrid_encode_margins(golden["hyb_x"], golden["hyb_packed"], hp)
    assert all(float(np.abs(v[g]).max()) == 0 for v in m.values() for g in (0, 1))
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((3000, 128)) * rng.lognormal(0, 0.5, (3000, 1))).astype(np.float32)
    p = O.hybrid_encode(x, hp)
    m = O.hybrid_encode_margins(x, p, hp)
    for g in (0, 1):
        assert m["code_ulps"][g].max() <= 4 and m["sign_ulps"][g].max() <= 4
        assert np.abs(m["norm_steps"][g]).max() <= 1 and np.abs(m["rnorm_steps"][g]).max() <= 1
    bad = p.copy()
    bad[7, 3] ^= 0x10          # a group-0 code bit
    bad[9, 25] ^= 0x01         # a group-0 sign bit
    bad[11, 40] ^= 0x40        # a group-1 code bit
    bad[13, 61] ^= 0x04        # group-1 norm, fp16 high byte
    m = O.hybrid_encode_margins(x, bad, hp)
    assert m["code_ulps"][0][7].max() > 1e3 and m["sign_ulps"][0][9].max() > 1e3
    assert m["code_ulps"][1][11].max() > 1e3 and abs(int(m["norm_steps"][1][13])) > 100
    assert m["code_ulps"][0][8].max() == 0 and m["sign_ulps"][1][9].max() == 0


def test_boundary_distance_counts_ulps_of_the_largest_term_under_cancellation():
    """A value 4e-9 above the boundary at 0 that came out of terms of 2e-2 is two float32 ulps of those terms
    away from it, not millions of ulps of itself; away from cancellation the floor changes nothing."""
    b = np.array([-0.02, 0.0, 0.02])
    y = np.array([3.99e-9, 0.0200001])
    plain = O.boundary_ulp_distance(y, b)
    assert plain[0] > 1e6 and abs(plain[1] - 1e-7 / np.spacing(np.float32(0.0200001))) < 1e-3
    floored = O.boundary_ulp_distance(y, b, floor=np.array([0.018, 0.018]))
    assert abs(floored[0] - 3.99e-9 / np.spacing(np.float32(0.018))) < 1e-6 and floored[0] < 3
    assert floored[1] == plain[1]


# ---- hybrid, mode tq25 -------------------------------------------------------------------------
def tq25_params(tq25):
    books = ((tq25["g0_centroids"], tq25["g0_boundaries"]), (tq25["g1_centroids"], tq25["g1_boundaries"]))
    return O.HybridParams(tq25["g0_had"], tq25["g1_had"], tq25["g0_qjl"], tq25["g1_qjl"], codebooks=books, mode="tq25")


def test_tq25_oracle_reproduces_the_reference_rows(tq25):
    """Rows and decoded vectors of the reference itself (groups of 32 and 96 coordinates, 44-byte rows): the
    oracle's encode and decode give them bit for bit, for one head and for two."""
    hp = tq25_params(tq25)
    assert hp.packed_dim == int(tq25["packed_dim"]) == 44 and hp.group_bytes == (16, 28)
    assert np.array_equal(O.hybrid_encode(tq25["x"], hp), tq25["packed"])
    assert np.array_equal(O.hybrid_decode(tq25["packed"], hp), tq25["decoded"])
    assert np.array_equal(O.hybrid_encode(tq25["x_heads2"], hp), tq25["packed_heads2"])
    assert np.array_equal(O.hybrid_decode(tq25["packed_heads2"], hp), tq25["decoded_heads2"])
    # the grid iteration: centroids bit for bit; the middle boundary of a symmetric book is float64 summation
    # noise in the reference (0.0 and -2^-57 here) and in the oracle's restatement alike
    for nm, (d, b) in (("g0", (32, 2)), ("g1", (96, 1))):
        c, bd = O.dimension_aware_codebook(d, b)
        assert np.array_equal(c, tq25[nm + "_centroids"])
        mid = len(bd) // 2
        assert np.array_equal(np.delete(bd, mid), np.delete(tq25[nm + "_boundaries"], mid))
        assert abs(float(bd[mid])) < 1e-16 and abs(float(tq25[nm + "_boundaries"][mid])) < 1e-16
    m = O.hybrid_encode_margins(tq25["x"], tq25["packed"], hp)
    assert all(float(np.abs(v[g]).max()) == 0 for v in m.values() for g in (0, 1))


def test_transform_of_96_points_is_two_blocks():
    """fwht_general on 96 points = a 64-point and a 32-point Hadamard matrix side by side; the structured
    transform divides both by sqrt(96), so forward-then-inverse scales the blocks by 64/96 and 32/96 (the
    reference's transform is not unitary at this length)."""
    rng = np.random.default_rng(4)
    x = rng.standard_normal((6, 96)).astype(np.float32)
    H = O._hadamard_matrix(96)
    assert np.array_equal(H[:64, 64:], np.zeros((64, 32))) and np.array_equal(H, H.T)
    assert np.array_equal(H[:64, :64] @ H[:64, :64], 64 * np.eye(64)) and np.array_equal(H[64:, 64:] @ H[64:, 64:], 32 * np.eye(32))
    assert np.allclose(O.fwht_general(x), x @ H, atol=1e-4)
    assert np.array_equal(O.fwht_general(x[:, :64]), O.fwht(x[:, :64]))
    s = np.sign(rng.standard_normal(96)).astype(np.float32)
    back = O.structured_hadamard(O.structured_hadamard(x, s), s, inverse=True)
    assert np.allclose(back[:, :64], x[:, :64] * (64 / 96), atol=1e-5)
    assert np.allclose(back[:, 64:], x[:, 64:] * (32 / 96), atol=1e-5)


def test_tq25_margins_catch_defects(tq25):
    hp = tq25_params(tq25)
    rng = np.random.default_rng(10)
    x = (rng.standard_normal((2000, 128)) * rng.lognormal(0, 0.5, (2000, 1))).astype(np.float32)
    p = O.hybrid_encode(x, hp)
    m = O.hybrid_encode_margins(x, p, hp)
    for g in (0, 1):
        assert m["code_ulps"][g].max() <= 4 and m["sign_ulps"][g].max() <= 4
        assert np.abs(m["norm_steps"][g]).max() <= 1 and np.abs(m["rnorm_steps"][g]).max() <= 1
    bad = p.copy()
    bad[7, 3] ^= 0x40          # a group-0 code bit
    bad[9, 9] ^= 0x01          # a group-0 sign bit
    bad[11, 20] ^= 0x40        # a group-1 code bit
    bad[12, 33] ^= 0x02        # a group-1 sign bit
    bad[13, 41] ^= 0x04        # group-1 norm, fp16 high byte
    m = O.hybrid_encode_margins(x, bad, hp)
    assert m["code_ulps"][0][7].max() > 1e3 and m["sign_ulps"][0][9].max() > 1e3
    assert m["code_ulps"][1][11].max() > 1e3 and m["sign_ulps"][1][12].max() > 1e3
    assert abs(int(m["norm_steps"][1][13])) > 100
    assert m["code_ulps"][0][8].max() == 0 and m["sign_ulps"][1][9].max() == 0

"""The numpy oracle against the vectors the reference itself produced (CPU only)."""
import os

import numpy as np
import pytest

from oracle import tq_oracle as O
from tests.util import code_mismatch_report


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_codebooks_equal_reference(golden, bits):
    c, b, _ = O.get_codebook(128, bits)
    assert np.array_equal(c, golden[f"centroids_b{bits}"])
    assert np.array_equal(b, golden[f"boundaries_b{bits}"])


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_encode_matches_reference(golden, bits):
    R = golden["rotation_d128_seed42"]
    _, b, _ = O.get_codebook(128, bits)
    packed, norms = O.encode(golden["enc_x"], R, b, bits)
    ref_p, ref_n = golden[f"enc_packed_b{bits}"], golden[f"enc_norms_b{bits}"]
    assert packed.shape == ref_p.shape and packed.dtype == np.uint8
    ca, cb = O._UNPACK[bits](packed, 128), O._UNPACK[bits](ref_p, 128)
    n, max_ulps, hist = code_mismatch_report(ca, cb, O.rotate_unit_f64(golden["enc_x"], R), b, O)
    # two float32 summation orders (numpy's BLAS, torch's MKL) may disagree only on values that
    # sit within a few float32 ulps of a decision boundary, and then by one code step
    assert n <= 2 and max_ulps <= 16 and hist.get("max_code_step", 1) == 1, (n, max_ulps, hist)
    nz = ref_n > 0
    assert np.max(np.abs(norms[nz] - ref_n[nz]) / ref_n[nz]) < 1e-6
    assert norms[5] == 0 and ref_n[5] == 0
    # the all-zero vector: y == boundary[mid] == 0.0 exactly, tie goes to the lower bin
    mid = (1 << bits) // 2 - 1
    assert np.all(cb[5] == mid) and np.all(ca[5] == mid)


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_decode_matches_reference(golden, bits):
    R = golden["rotation_d128_seed42"]
    c, _, _ = O.get_codebook(128, bits)
    d = O.decode(golden[f"enc_packed_b{bits}"], golden[f"enc_norms_b{bits}"], R, c, bits)
    ref = golden[f"dec_b{bits}"]
    assert d.dtype == np.float16
    # fp16 outputs: equal except where the float32 value sits on an fp16 rounding boundary
    assert np.mean(d == ref) > 0.999
    assert np.max(np.abs(d.astype(np.float32) - ref.astype(np.float32))) <= 2e-3


def test_encode_other_dtypes_and_dims(golden):
    R = golden["rotation_d128_seed42"]
    _, b, _ = O.get_codebook(128, 4)
    for x, pk, nk in ((golden["enc_x_f32"], "enc_packed_f32_b4", "enc_norms_f32_b4"),
                      (golden["enc_x_bf16_as_f32"], "enc_packed_bf16_b4", "enc_norms_bf16_b4")):
        p, n = O.encode(x, R, b, 4)
        assert np.mean(p == golden[pk]) > 0.999
        assert np.allclose(n, golden[nk], rtol=1e-6)
    R64 = golden["rotation_d64_seed42"]
    c64, b64, _ = O.get_codebook(64, 4)
    p, n = O.encode(golden["enc_x_d64"], R64, b64, 4)
    assert np.mean(p == golden["enc_packed_d64_b4"]) > 0.999
    d = O.decode(golden["enc_packed_d64_b4"], golden["enc_norms_d64_b4"], R64, c64, 4)
    assert np.max(np.abs(d.astype(np.float32) - golden["dec_d64_b4"].astype(np.float32))) <= 2e-3


@pytest.mark.parametrize("max_blocks,suffix", [(6, ""), (4, "_max4")])
def test_kv_update_scatter_semantics(golden, max_blocks, suffix):
    R = golden["rotation_d128_seed42"]
    _, b, _ = O.get_codebook(128, 4)
    kp = np.zeros((6, 16, 2, 64), np.uint8)
    kn = np.zeros((6, 16, 2), np.float32)
    O.kv_update(golden["upd_x"], golden["upd_slots"], kp, kn, R, b, 16, max_blocks, bits=4)
    assert np.mean(kp == golden["upd_packed" + suffix]) > 0.9999
    assert np.allclose(kn, golden["upd_norms" + suffix], rtol=1e-6)
    # skipped tokens leave zeros: same set of written rows
    assert np.array_equal(kn != 0, golden["upd_norms" + suffix] != 0)


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_paged_attention_matches_reference(golden, bits):
    R = golden["rotation_d128_seed42"]
    c, _, _ = O.get_codebook(128, bits)
    tables = golden["attn_tables"].copy()
    args = (golden["attn_q"], golden[f"attn_kp_b{bits}"], golden[f"attn_kn_b{bits}"],
            golden[f"attn_vp_b{bits}"], golden[f"attn_vn_b{bits}"], tables, golden["attn_ctx"],
            R, c, bits)
    ref = golden[f"attn_out_b{bits}"].astype(np.float32)
    loop = O.paged_attention_loop(*args).astype(np.float32)     # never touches the 10**6 padding entry
    vec = O.paged_attention(*args).astype(np.float32)
    assert np.all(ref[0] == 0) and np.all(loop[0] == 0) and np.all(vec[0] == 0)   # ctx == 0
    assert np.max(np.abs(loop - ref)) <= 1e-3   # half an fp16 ulp at |out| < 4
    assert np.max(np.abs(vec - ref)) <= 1e-3
    v64 = O.paged_attention(*args, dtype=np.float64, cast_output=False)
    assert np.max(np.abs(v64 - ref)) <= 1.5e-3


def test_hybrid_tables_and_codec_match_reference(golden):
    for bits in (3, 2):
        c, b = O.dimension_aware_codebook(64, bits)
        assert np.array_equal(c, golden[f"hyb_centroids_64_{bits}"])
        # the middle boundary is 0 up to float64 summation noise (|b| < 1e-15) in both
        assert np.allclose(b, golden[f"hyb_boundaries_64_{bits}"], rtol=0, atol=1e-15)
    books = tuple((golden[f"hyb_centroids_64_{k}"], golden[f"hyb_boundaries_64_{k}"]) for k in (3, 2))
    hp = O.HybridParams(golden["hyb_g0_had_signs"], golden["hyb_g1_had_signs"],
                        golden["hyb_g0_qjl_signs"], golden["hyb_g1_qjl_signs"], codebooks=books)
    packed = O.hybrid_encode(golden["hyb_x"], hp)
    assert np.array_equal(packed, golden["hyb_packed"])
    assert np.array_equal(O.hybrid_encode(golden["hyb_x_heads2"], hp), golden["hyb_packed_heads2"])
    dec = O.hybrid_decode(golden["hyb_packed"], hp)
    assert np.array_equal(dec, golden["hyb_decoded"])
    assert np.array_equal(O.hybrid_decode(golden["hyb_packed_heads2"], hp), golden["hyb_decoded_heads2"])


def test_tri_matches_reference(golden):
    th = golden["theta_d128_base1e6"]
    # numpy's and torch's float32 pow may differ in the last place
    assert np.max(np.abs(O.rope_frequencies(128, 1e6) - th) / th) < 2e-7
    assert np.array_equal(O.rope_frequencies(32, 1e4), golden["theta_d32_base1e4"])
    for nm, src in (("k", golden["tri_keys"]), ("v", golden["tri_vals"])):
        i, p, s = O.spectral_encode(src, 12)
        assert np.array_equal(i, golden[f"tri_{nm}_indices"])
        assert np.array_equal(p, golden[f"tri_{nm}_packed"])
        assert np.array_equal(s, golden[f"tri_{nm}_scales"])
    ke = tuple(golden[f"tri_k_{n}"] for n in ("indices", "packed", "scales"))
    ve = tuple(golden[f"tri_v_{n}"] for n in ("indices", "packed", "scales"))
    sc = O.tri_scores(golden["tri_q"], *ke, th, golden["tri_qpos"], golden["tri_kpos"])
    assert np.max(np.abs(sc - golden["tri_scores_explicit_pos"])) < 2e-6
    o1 = O.tri_decode_step(golden["tri_q"], ke, ve, th)
    assert np.max(np.abs(o1 - golden["tri_out_default_pos"])) < 1e-6
    o2 = O.tri_decode_step(golden["tri_q"], ke, ve, th, golden["tri_qpos"], golden["tri_kpos"])
    assert np.max(np.abs(o2 - golden["tri_out_explicit_pos"])) < 1e-6


@pytest.mark.parametrize("bits,pre", [(8, True), (16, True), (4, False), (8, False), (16, False)])
def test_tri_coefficient_widths_and_post_rope_match_reference(golden, tri_widths, bits, pre):
    """Encodings bit for bit; scores and outputs to a few float32 ulps of their sums (numpy's and torch's
    cos / sin / exp and summation order differ in the last place)."""
    g, th = tri_widths, golden["theta_d128_base1e6"]
    tag = f"b{bits}_{'pre' if pre else 'post'}"
    for nm, src in (("k", g["keys"]), ("v", g["vals"])):
        i, p, s = O.spectral_encode(src, 12, bits)
        assert np.array_equal(i, g[f"enc_b{bits}_{nm}_indices"])
        assert p.dtype == g[f"enc_b{bits}_{nm}_packed"].dtype and np.array_equal(p, g[f"enc_b{bits}_{nm}_packed"])
        assert np.array_equal(s, g[f"enc_b{bits}_{nm}_scales"])
    ke = tuple(g[f"enc_b{bits}_k_{n}"] for n in ("indices", "packed", "scales"))
    ve = tuple(g[f"enc_b{bits}_v_{n}"] for n in ("indices", "packed", "scales"))
    sc = O.tri_scores(g["q"], *ke, th, g["qpos"], g["kpos"], bits, pre)
    assert np.max(np.abs(sc - g[f"scores_{tag}"])) < 2e-6
    o = O.tri_decode_step(g["q"], ke, ve, th, g["qpos"], g["kpos"], bits, pre)
    assert np.max(np.abs(o - g[f"out_{tag}"])) < 1e-6
    o = O.tri_decode_step(g["q"], ke, ve, th, None, None, bits, pre)
    assert np.max(np.abs(o - g[f"out_default_pos_{tag}"])) < 1e-6
    if not pre:      # positions play no part in the plain dot product
        assert np.array_equal(g[f"out_{tag}"], g[f"out_default_pos_{tag}"])


# ---- block selector (vectors written by tests/golden/make_golden_block_selector.py) -------------
@pytest.fixture(scope="module")
def bsel():
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden_block_selector.npz"))


def test_block_representatives_golden(bsel):
    MB, H, PD = 12, 2, 64
    acc_e = np.zeros((MB, H, PD), np.float32); acc_o = np.zeros_like(acc_e)
    rep_e = np.zeros_like(acc_e); rep_o = np.zeros_like(acc_e)
    counts = np.zeros((MB, H), np.int16)
    for call in range(3):
        bi = bsel[f"rep_bi_{call}"]
        O.block_rep_update(acc_e, acc_o, counts, bi, bsel[f"rep_kp_{call}"], bsel[f"rep_kn_{call}"], bsel["centroids"])
        O.block_rep_finalize(acc_e, acc_o, counts, rep_e, rep_o, np.unique(bi))
        assert np.array_equal(counts, bsel[f"rep_counts_after_{call}"])
        # the reference adds in torch's scatter order, the oracle in input order: a few ulps of a sum
        np.testing.assert_allclose(rep_e, bsel[f"rep_even_after_{call}"], rtol=2e-6, atol=1e-7)
        np.testing.assert_allclose(rep_o, bsel[f"rep_odd_after_{call}"], rtol=2e-6, atol=1e-7)
    assert np.all(bsel["rep_counts_after_2"][10:] == 0) and np.all(bsel["rep_even_after_2"][10:] == 0)


def test_block_scores_and_selection_golden(bsel):
    sc = O.block_scores(bsel["sel_q_even"], bsel["sel_q_odd"], bsel["sel_rep_even"], bsel["sel_rep_odd"],
                        bsel["sel_bt"], bsel["sel_ctx"], 4, 16)
    ref = bsel["sel_scores"]
    assert np.array_equal(np.isneginf(sc), np.isneginf(ref))
    fin = np.isfinite(ref)
    assert np.max(np.abs(sc[fin] - ref[fin])) <= 2e-5
    nb = (bsel["sel_ctx"] + 15) // 16
    for tag, ms, sinks, recents in (("10", 10, 2, 2), ("40", 40, 2, 2), ("120", 120, 2, 2), ("12_s1r3", 12, 1, 3)):
        fbt, fcl = O.block_select(ref, bsel["sel_bt"], bsel["sel_ctx"], 16, ms, sinks, recents)
        rbt, rcl = bsel[f"sel_fbt_{tag}"], bsel[f"sel_fcl_{tag}"]
        assert np.array_equal(fcl, rcl) and fbt.shape == rbt.shape
        k = min(ms, bsel["sel_bt"].shape[1])
        for s in range(fbt.shape[0]):
            m = min(k, int(nb[s]))          # beyond the valid blocks the reference's choice among -inf columns is arbitrary
            assert np.array_equal(fbt[s, :m], rbt[s, :m])
        assert np.all(fbt[:, k:] == 0) and np.all(rbt[:, k:] == 0)
    assert int(bsel["cls_max_selected"]) == 30
    fbt, fcl = O.block_select(ref, bsel["sel_bt"], bsel["sel_ctx"], 16, 30)
    assert np.array_equal(fcl, bsel["cls_fcl"])
    for s in range(3):
        m = min(30, int(nb[s]))
        assert np.array_equal(fbt[s, :m], bsel["cls_fbt"][s, :m])


def test_block_select_orders_nan_and_zeros_like_topk():
    """torch.topk, which the reference's selection is (block_selector.py:205-207), ranks a NaN above everything
    and treats the two zeros as equal: the oracle's selection on scores with NaNs, +-0 and otherwise distinct
    values equals topk's wherever topk's answer does not depend on its choice among equal keys."""
    import torch
    rng = np.random.default_rng(5)
    compared = 0
    for _ in range(300):
        S, B, bs = 3, int(rng.integers(1, 80)), 16
        ms, sinks, recents = int(rng.integers(1, B + 3)), int(rng.integers(0, 3)), int(rng.integers(0, 3))
        sc = (rng.permutation(S * B).reshape(S, B) - S * B // 2).astype(np.float32)      # distinct; one of them is 0
        sc[rng.random((S, B)) < 0.1] = np.nan
        sc[sc == 0] = -0.0 if rng.random() < 0.5 else 0.0
        ctx = rng.integers(0, B * bs + 1, S).astype(np.int64)
        table = np.tile(np.arange(B), (S, 1)).astype(np.int64)           # ids = columns: the selection can be read off
        fbt, _ = O.block_select(sc, table, ctx, bs, ms, sinks, recents)
        t = torch.from_numpy(sc.copy())
        nb = (torch.from_numpy(ctx) + bs - 1) // bs
        col = torch.arange(B)[None]
        valid = col < nb[:, None]
        t[((col < sinks) | (col >= nb[:, None] - recents)) & valid] = float("inf")
        t[~valid] = float("-inf")
        k = min(ms, B)
        idx = t.topk(k, dim=1, sorted=False)[1].sort(dim=1)[0].numpy()
        for s in range(S):
            row = t[s].numpy().astype(np.float64)
            key = np.where(np.isnan(row), np.inf, np.clip(row, -1e300, 1e300))      # NaN above +inf
            kth = np.sort(key)[::-1][k - 1]
            if int(np.sum(key >= kth)) != k:
                continue                                             # topk chooses among equal keys at the cut
            assert np.array_equal(np.sort(idx[s]), fbt[s, :k]), (row, idx[s], fbt[s])
            compared += 1
    assert compared > 300

"""HIP codec kernels (through the C ABI) against the oracle and the reference's own vectors."""
import numpy as np
import pytest
import torch

import aitherkvcache_amd as akv
from aitherkvcache_amd import _lib, triton_ops
from oracle import tq_oracle as O
from tests.util import kv_like, code_mismatch_report, check_codes, MAX_ULPS

pytestmark = pytest.mark.gpu

def make_tq(golden, dev, bits, d=128):
    tq = akv.TurboQuant(head_dim=d, bits=bits, device=str(dev))
    tq.rotation = torch.from_numpy(golden[f"rotation_d{d}_seed42"]).to(dev)   # the reference's matrix
    return tq


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_encode_decode_golden(golden, dev, bits):
    tq = make_tq(golden, dev, bits)
    x = golden["enc_x"]
    packed, norms = tq.encode(torch.from_numpy(x).to(dev))
    assert packed.dtype == torch.uint8 and packed.shape == (96, tq._packed_dim)
    assert norms.dtype == torch.float32 and norms.shape == (96,)
    check_codes(packed.cpu().numpy(), norms.cpu().numpy(), x, golden["rotation_d128_seed42"], bits,
                golden[f"enc_packed_b{bits}"], golden[f"enc_norms_b{bits}"])
    # zero vector: ties at boundary 0.0 go to the lower bin (0x77.. at 4-bit), norm 0
    mid = (1 << bits) // 2 - 1
    assert np.all(O._UNPACK[bits](packed[5:6].cpu().numpy(), 128) == mid)
    dec = tq.decode(torch.from_numpy(golden[f"enc_packed_b{bits}"]).to(dev),
                    torch.from_numpy(golden[f"enc_norms_b{bits}"]).to(dev))
    assert dec.dtype == torch.float16
    ref = golden[f"dec_b{bits}"].astype(np.float32)
    got = dec.cpu().numpy().astype(np.float32)
    assert np.max(np.abs(got - ref)) <= 2e-3
    assert np.mean(got == ref) > 0.995


@pytest.mark.parametrize("dtype,key", [(torch.float32, "f32"), (torch.bfloat16, "bf16")])
def test_encode_other_input_dtypes(golden, dev, dtype, key):
    tq = make_tq(golden, dev, 4)
    src = golden["enc_x_f32"] if key == "f32" else golden["enc_x_bf16_as_f32"]
    x = torch.from_numpy(src).to(dev).to(dtype)
    packed, norms = tq.encode(x)
    check_codes(packed.cpu().numpy(), norms.cpu().numpy(), src, golden["rotation_d128_seed42"], 4,
                golden[f"enc_packed_{key}_b4"], golden[f"enc_norms_{key}_b4"])


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_encode_bfloat16_wide_range_vs_oracle(golden, dev, bits):
    """bfloat16 rows go through a per-row power-of-two scaling: rows of very large, very small and
    mixed magnitudes must give the oracle's codes (the oracle sees the same bfloat16 values)."""
    rng = np.random.default_rng(77 + bits)
    n = 2048 + 17
    x = rng.standard_normal((n, 128)).astype(np.float32)
    scale = np.exp2(rng.integers(-40, 40, size=n)).astype(np.float32)         # rows from 2^-40 to 2^40
    x *= scale[:, None]
    x[::7] *= np.exp2(rng.integers(-20, 1, size=(len(x[::7]), 128))).astype(np.float32)   # wide range inside a row
    x[3] = 0.0
    xb = torch.from_numpy(x).to(torch.bfloat16)
    tq = make_tq(golden, dev, bits)
    packed, norms = tq.encode(xb.to(dev))
    check_codes(packed.cpu().numpy(), norms.cpu().numpy(), xb.float().numpy(), golden["rotation_d128_seed42"], bits)
    # squares that overflow float32: norm inf, unit vector 0, every code is #{b < 0}; an infinite
    # element makes the rotated vector NaN: every code is the last level (searchsorted puts NaN last)
    y = torch.full((2, 128), 2.0 ** 70, dtype=torch.bfloat16)
    y[1, 5] = float("inf")
    packed, norms = tq.encode(y.to(dev))
    codes = O._UNPACK[bits](packed.cpu().numpy(), 128)
    assert np.all(codes[0] == (1 << bits) // 2 - 1) and np.all(codes[1] == (1 << bits) - 1)
    assert np.all(np.isinf(norms.cpu().numpy()))


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_encode_float32_wide_range_vs_oracle(golden, dev, bits):
    """float32 rows are scaled by a power of two and split into two float16 terms for the matrix cores: rows of
    very large, very small and mixed magnitudes, a zero row, odd row counts and strided rows must give the
    oracle's codes (every differing code within the boundary allowance of check_codes)."""
    rng = np.random.default_rng(177 + bits)
    n = 20000 + 13
    x = rng.standard_normal((n, 128)).astype(np.float32)
    scale = np.exp2(rng.integers(-60, 60, size=n)).astype(np.float32)         # rows from 2^-60 to 2^60
    x *= scale[:, None]
    x[::7] *= np.exp2(rng.integers(-30, 1, size=(len(x[::7]), 128))).astype(np.float32)   # wide range inside a row
    x[3] = 0.0
    x[4] = 0.0
    x[4, 17] = -3.25                                                           # one non-zero element
    tq = make_tq(golden, dev, bits)
    xt = torch.from_numpy(x).to(dev)
    packed, norms = tq.encode(xt)
    check_codes(packed.cpu().numpy(), norms.cpu().numpy(), x, golden["rotation_d128_seed42"], bits)
    # rows with a stride (a column slice of a wider tensor) and a leading batch shape
    wide = torch.zeros(50, 3, 256, device=dev)
    wide[..., 64:192] = xt[:150].reshape(50, 3, 128)
    p2, n2 = tq.encode(wide[..., 64:192])
    assert torch.equal(p2.reshape(150, -1), packed[:150]) and torch.equal(n2.reshape(150), norms[:150])
    # overflowing squares, an infinity, a NaN
    y = torch.full((3, 128), 2.0 ** 70, dtype=torch.float32)
    y[1, 5] = float("inf")
    y[2, 100] = float("nan")
    packed, norms = tq.encode(y.to(dev))
    codes = O._UNPACK[bits](packed.cpu().numpy(), 128)
    assert np.all(codes[0] == (1 << bits) // 2 - 1) and np.all(codes[1] == (1 << bits) - 1) and np.all(codes[2] == (1 << bits) - 1)
    assert np.all(np.isinf(norms.cpu().numpy()[:2])) and np.isnan(norms.cpu().numpy()[2])


def test_head_dim_64(golden, dev):
    tq = make_tq(golden, dev, 4, d=64)
    x = golden["enc_x_d64"]
    packed, norms = tq.encode(torch.from_numpy(x).to(dev))
    check_codes(packed.cpu().numpy(), norms.cpu().numpy(), x, golden["rotation_d64_seed42"], 4,
                golden["enc_packed_d64_b4"], golden["enc_norms_d64_b4"], d=64)
    dec = tq.decode(torch.from_numpy(golden["enc_packed_d64_b4"]).to(dev),
                    torch.from_numpy(golden["enc_norms_d64_b4"]).to(dev)).cpu().numpy()
    assert np.max(np.abs(dec.astype(np.float32) - golden["dec_d64_b4"].astype(np.float32))) <= 2e-3


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("d", [256, 512])
def test_wide_heads_codec_and_attention_vs_oracle(dev, bits, d):
    """head_dim 256 and 512 (the reference's quantizer takes every power of two, quantizer.py:78-81, and its
    backend lists 512, vllm/backend.py:308-309): flat encode / decode, the paged write and decode attention
    against the oracle, with the matrix the quantizer itself draws for the dimension."""
    tq = akv.TurboQuant(head_dim=d, bits=bits, device=str(dev))
    R = tq.rotation.cpu().numpy()
    rng = np.random.default_rng(d + bits)
    x = kv_like(rng, (300, d))
    packed, norms = tq.encode(torch.from_numpy(x).to(dev))
    assert packed.shape == (300, d * bits // 8)
    check_codes(packed.cpu().numpy(), norms.cpu().numpy(), x, R, bits, d=d)
    c, b, _ = O.get_codebook(d, bits)
    dec = tq.decode(packed, norms).cpu().numpy().astype(np.float32)
    ref = O.decode(packed.cpu().numpy(), norms.cpu().numpy(), R, c, bits)
    assert np.max(np.abs(dec - ref.astype(np.float32))) <= 2e-3 * max(1.0, np.abs(ref).max() / 4)
    # paged write + decode attention (GQA 4:1, ragged contexts, permuted tables)
    NB, BS, KVH, QH = 12, 16, 2, 8
    P = tq._packed_dim
    keys, vals = kv_like(rng, (NB * BS, KVH, d)), kv_like(rng, (NB * BS, KVH, d))
    kp = torch.zeros(NB, BS, KVH, P, dtype=torch.uint8, device=dev)
    vp = torch.zeros_like(kp)
    kn = torch.zeros(NB, BS, KVH, device=dev)
    vn = torch.zeros_like(kn)
    slots = torch.from_numpy(rng.permutation(NB * BS)).to(dev)
    akv.fused_kv_update(torch.from_numpy(keys).to(dev), slots, kp, kn, tq.rotation, tq.boundaries_inner, bits, BS)
    akv.fused_kv_update(torch.from_numpy(vals).to(dev), slots, vp, vn, tq.rotation, tq.boundaries_inner, bits, BS)
    ref_p = np.zeros((NB, BS, KVH, P), np.uint8)
    ref_n = np.zeros((NB, BS, KVH), np.float32)
    O.kv_update(keys, slots.cpu().numpy(), ref_p, ref_n, R, b, BS, 0, bits)
    assert np.mean(kp.cpu().numpy() == ref_p) > 0.9999 and np.allclose(kn.cpu().numpy(), ref_n, rtol=1e-6)
    ctx = np.array([0, 1, 17, 150, NB * BS], dtype=np.int64)
    tables = np.stack([rng.permutation(NB) for _ in ctx]).astype(np.int32)
    q = rng.standard_normal((len(ctx), QH, d)).astype(np.float16)
    out = akv.TQPagedAttention(tq, QH).forward(torch.from_numpy(q).to(dev), kp, kn, vp, vn,
                                               torch.from_numpy(tables).to(dev), torch.from_numpy(ctx).to(dev))
    want = O.paged_attention(q, kp.cpu().numpy(), kn.cpu().numpy(), vp.cpu().numpy(), vn.cpu().numpy(), tables, ctx,
                             R, c, bits, dtype=np.float64, cast_output=False)
    got = out.cpu().numpy().astype(np.float64)
    assert np.all(got[0] == 0) and np.all(np.abs(got - want) <= 2e-3 + 2.0 ** -11 * np.abs(want))


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("n", [1, 31, 33, 4097])
def test_encode_ragged_sizes_vs_oracle(golden, dev, bits, n):
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(1000 + n + bits)
    x = kv_like(rng, (n, 128))
    packed, norms = tq.encode(torch.from_numpy(x).to(dev))
    check_codes(packed.cpu().numpy(), norms.cpu().numpy(), x, golden["rotation_d128_seed42"], bits)
    c, _, _ = O.get_codebook(128, bits)
    dec = tq.decode(packed, norms).cpu().numpy().astype(np.float32)
    ref = O.decode(packed.cpu().numpy(), norms.cpu().numpy(), golden["rotation_d128_seed42"], c, bits)
    assert np.max(np.abs(dec - ref.astype(np.float32))) <= 2e-3 * max(1.0, np.abs(ref).max() / 4)
    # float16 results almost always round the same way as the float32 oracle's
    assert np.mean(dec == ref.astype(np.float16).astype(np.float32)) > 0.99


def test_batch_shapes_and_empty(golden, dev):
    tq = make_tq(golden, dev, 4)
    x = torch.randn(2, 3, 5, 128, device=dev, dtype=torch.float16)
    p, n = tq.encode(x)
    assert p.shape == (2, 3, 5, 64) and n.shape == (2, 3, 5)
    assert tq.decode(p, n).shape == (2, 3, 5, 128)
    p1, n1 = tq.encode(x[0, 0, 0])
    assert p1.shape == (64,) and n1.shape == ()
    assert torch.equal(p1, p[0, 0, 0]) and torch.equal(n1, n[0, 0, 0])
    pe, ne = tq.encode(torch.zeros(0, 128, device=dev, dtype=torch.float16))
    assert pe.shape == (0, 64) and ne.shape == (0,)
    assert tq.decode(pe, ne).shape == (0, 128)
    # a strided view (every other row) encodes like its contiguous copy
    big = torch.randn(64, 256, device=dev, dtype=torch.float16)
    pv, nv = tq.encode(big[:, :128])
    pc, nc = tq.encode(big[:, :128].contiguous())
    assert torch.equal(pv, pc) and torch.equal(nv, nc)


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_quantize_pack_and_unpack_lookup_exact(golden, dev, bits):
    """Given the same rotated values these two are pure integer work: bit-exact."""
    c, b, _ = O.get_codebook(128, bits)
    rng = np.random.default_rng(5)
    y = rng.normal(0, 0.09, size=(257, 128)).astype(np.float32)
    y[0, :len(b)] = b                               # exact ties
    y[1, :len(b)] = np.nextafter(b, np.float32(np.inf))
    y[2] = 0.0
    got = triton_ops.hip_quantize(torch.from_numpy(y).to(dev), torch.from_numpy(b).to(dev), bits)
    want = O._PACK[bits](O.quantize(y, b, bits))
    assert np.array_equal(got.cpu().numpy(), want)
    back = triton_ops.hip_dequantize(got, torch.from_numpy(c).to(dev), 128, bits).cpu().numpy()
    assert np.array_equal(back, c[O._UNPACK[bits](want, 128).astype(np.int64)])
    if bits == 4:
        assert torch.equal(triton_ops.triton_quantize_4bit(torch.from_numpy(y).to(dev), torch.from_numpy(b).to(dev)), got)


@pytest.mark.parametrize("max_blocks,suffix", [(0, ""), (4, "_max4")])
def test_paged_update_golden(golden, dev, max_blocks, suffix):
    tq = make_tq(golden, dev, 4)
    kp = torch.zeros(6, 16, 2, 64, dtype=torch.uint8, device=dev)
    kn = torch.zeros(6, 16, 2, device=dev)
    akv.fused_tq4_kv_update(torch.from_numpy(golden["upd_x"]).to(dev),
                            torch.from_numpy(golden["upd_slots"]).to(dev), kp, kn, tq.rotation,
                            tq.boundaries_inner, block_size=16, max_blocks=max_blocks)
    ref_p, ref_n = golden["upd_packed" + suffix], golden["upd_norms" + suffix]
    assert np.array_equal(kn.cpu().numpy() != 0, ref_n != 0)          # same tokens skipped
    written = ref_n != 0
    x = golden["upd_x"]
    # rows in slot order for the ulp accounting
    slots = golden["upd_slots"]
    ok = (slots >= 0) & (slots // 16 < (max_blocks or 6))
    check_codes(kp.cpu().numpy()[slots[ok] // 16, slots[ok] % 16], kn.cpu().numpy()[slots[ok] // 16, slots[ok] % 16],
                x[ok], golden["rotation_d128_seed42"], 4,
                ref_p[slots[ok] // 16, slots[ok] % 16], ref_n[slots[ok] // 16, slots[ok] % 16])
    assert np.all(kp.cpu().numpy()[~written] == 0)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("itype", [torch.int64, torch.int32])
def test_paged_update_strided_cache(golden, dev, bits, itype):
    """The serving layout: uint8 [blocks, 2, bs, heads, packed + 4] with K = [:, 0], V = [:, 1];
    rows are only 4-byte aligned and norms live in a [layers, blocks, bs, heads] tensor."""
    tq = make_tq(golden, dev, bits)
    P = tq._packed_dim
    NB, BS, H, T = 8, 16, 4, 50
    rng = np.random.default_rng(77 + bits)
    cache = torch.full((NB, 2, BS, H, P + 4), 0xAB, dtype=torch.uint8, device=dev)
    norms = torch.zeros(3, NB, BS, H, device=dev)
    x = kv_like(rng, (T, H, 128))
    slots = rng.permutation(NB * BS)[:T].astype(np.int64)
    slots[::7] = -1
    akv.fused_kv_update(torch.from_numpy(x).to(dev), torch.from_numpy(slots).to(dev).to(itype),
                        cache[:, 1], norms[2], tq.rotation, tq.boundaries_inner, bits, block_size=BS)
    _, b, _ = O.get_codebook(128, bits)
    ref_p = np.full((NB, BS, H, P + 4), 0xAB, np.uint8)
    ref_n = np.zeros((NB, BS, H), np.float32)
    view = ref_p[..., :P]
    O.kv_update(x, slots, view, ref_n, golden["rotation_d128_seed42"], b, BS, 0, bits)
    got = cache.cpu().numpy()
    assert np.all(got[:, 0] == 0xAB)                                   # K half untouched
    assert np.all(got[:, 1][..., P:] == 0xAB)                          # spare bytes untouched
    ok = slots >= 0
    check_codes(got[:, 1][slots[ok] // BS, slots[ok] % BS][..., :P], norms[2].cpu().numpy()[slots[ok] // BS, slots[ok] % BS],
                x[ok], golden["rotation_d128_seed42"], bits)
    assert np.array_equal(norms[2].cpu().numpy() != 0, ref_n != 0)
    assert torch.all(norms[:2] == 0)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_small_paged_calls_share_a_step_among_wavefronts(golden, dev, bits, dtype, monkeypatch):
    """A paged call of a few thousand vectors runs the form in which eight wavefronts share a step of 16 vectors
    (an N-tile each); a larger call, and the same call with that form switched off, run a wavefront per step.
    Codes, norms and untouched rows are the same byte for byte -- also with a NaN vector, an infinite one, a zero one,
    skipped slots and a token count that is no multiple of 16."""
    tq = make_tq(golden, dev, bits)
    P = tq._packed_dim
    NB, BS, H = 40, 16, 8
    rng = np.random.default_rng(500 + bits)
    for T in (1, 37, 256, 600):                       # 8 .. 4,800 vectors: one step, ragged, a serving step, two steps per workgroup
        x = kv_like(rng, (T, H, 128)).astype(np.float32)
        if T > 30:
            x[3, 1, 5] = np.nan
            x[4, 2, 7] = np.inf
            x[5, 0] = 0
        xd = torch.from_numpy(x).to(dev).to(dtype)
        slots = rng.permutation(NB * BS)[:T].astype(np.int64)
        slots[::9] = -1
        sd = torch.from_numpy(slots).to(dev)
        outs = []
        for off in ("", "1"):
            if off:
                monkeypatch.setenv("AKV_ENCODE_NO_SPLIT", "1")
            else:
                monkeypatch.delenv("AKV_ENCODE_NO_SPLIT", raising=False)
            kp = torch.full((NB, BS, H, P + 4), 0xAB, dtype=torch.uint8, device=dev)
            kn = torch.full((NB, BS, H), -5.0, device=dev)
            akv.fused_kv_update(xd, sd, kp[..., :P], kn, tq.rotation, tq.boundaries_inner, bits, BS)
            outs.append((kp.cpu().numpy(), kn.cpu().numpy()))
        monkeypatch.delenv("AKV_ENCODE_NO_SPLIT", raising=False)
        assert np.array_equal(outs[0][0], outs[1][0]), (bits, dtype, T)
        assert np.array_equal(outs[0][1], outs[1][1], equal_nan=True), (bits, dtype, T)
        assert int(np.sum(outs[0][1] != -5.0)) == int(np.sum(slots >= 0)) * H
        # the same vectors through the flat entry point (TurboQuant.encode), with and without the shared steps
        flat = []
        for off in ("", "1"):
            if off:
                monkeypatch.setenv("AKV_ENCODE_NO_SPLIT", "1")
            else:
                monkeypatch.delenv("AKV_ENCODE_NO_SPLIT", raising=False)
            p_, n_ = tq.encode(xd.reshape(-1, 128))
            flat.append((p_.cpu().numpy(), n_.cpu().numpy()))
        monkeypatch.delenv("AKV_ENCODE_NO_SPLIT", raising=False)
        assert np.array_equal(flat[0][0], flat[1][0]) and np.array_equal(flat[0][1], flat[1][1], equal_nan=True)
        ok = slots >= 0
        assert np.array_equal(outs[0][0][slots[ok] // BS, slots[ok] % BS][..., :P], flat[0][0].reshape(T, H, P)[ok])


def test_fused_encode_and_store(golden, dev):
    class Cache:
        pass
    c = Cache()
    c.tq = make_tq(golden, dev, 4)
    c.block_size, c.max_blocks = 16, 4
    c.k_packed = torch.zeros(2, 4, 16, 2, 64, dtype=torch.uint8, device=dev)
    c.v_packed = torch.zeros_like(c.k_packed)
    c.k_norms = torch.zeros(2, 4, 16, 2, device=dev)
    c.v_norms = torch.zeros_like(c.k_norms)
    k = torch.randn(5, 2, 128, device=dev, dtype=torch.float16)
    v = torch.randn(5, 2, 128, device=dev, dtype=torch.float16)
    slots = torch.tensor([3, 17, 40, 63, 64], device=dev)      # 64 -> block 4 >= max_blocks: skipped
    akv.fused_encode_and_store(c, 1, k, v, slots)
    R = golden["rotation_d128_seed42"]
    _, bnd, _ = O.get_codebook(128, 4)
    for x, packed, norms in ((k, c.k_packed, c.k_norms), (v, c.v_packed, c.v_norms)):
        ref_p = np.zeros((4, 16, 2, 64), np.uint8)
        ref_n = np.zeros((4, 16, 2), np.float32)
        O.kv_update(x.cpu().numpy(), slots.cpu().numpy(), ref_p, ref_n, R, bnd, block_size=16, max_blocks=4, bits=4)
        written = ref_n > 0
        assert np.array_equal(norms[1].cpu().numpy() > 0, written)            # the same slots, nothing else
        check_codes(packed[1].cpu().numpy()[written], norms[1].cpu().numpy()[written],
                    x[:4].cpu().numpy().reshape(-1, 128), R, 4, ref_p[written], ref_n[written])
        assert np.all(packed[1].cpu().numpy()[~written] == 0)
    assert torch.all(c.k_packed[0] == 0) and int((c.k_norms[1] != 0).sum()) == 8


def test_rotation_argument_is_told_apart_by_layout_and_contents(golden, dev):
    """fused_kv_update keeps the prepared form of the matrix it is handed.  A transposed view shares address and
    version counter with its base; a matrix rewritten in place keeps its address; a new matrix may be given the
    address of a freed one: each call must encode with the matrix it was handed."""
    tq = make_tq(golden, dev, 4)
    R = golden["rotation_d128_seed42"]
    rng = np.random.default_rng(12)
    x = kv_like(rng, (64, 2, 128))
    slots = torch.arange(64, device=dev)
    _, bnd, _ = O.get_codebook(128, 4)

    def run(rot):
        packed = torch.zeros(4, 16, 2, 64, dtype=torch.uint8, device=dev)
        norms = torch.zeros(4, 16, 2, device=dev)
        akv.fused_kv_update(torch.from_numpy(x).to(dev), slots, packed, norms, rot, tq.boundaries_inner, 4, 16)
        ref_p = np.zeros((4, 16, 2, 64), np.uint8)
        ref_n = np.zeros((4, 16, 2), np.float32)
        Rh = rot.detach().float().cpu().numpy()
        O.kv_update(x, slots.cpu().numpy(), ref_p, ref_n, Rh, bnd, 16, 0, 4)
        assert np.mean(packed.cpu().numpy() == ref_p) > 0.999, "encoded with another matrix"

    rot = torch.from_numpy(R).to(dev)
    run(rot)
    run(rot.t())                         # same address, same version, other layout
    run(rot)
    rot.copy_(rot.flip(0))               # same address, rewritten
    run(rot)
    for seed in range(3):                # fresh matrices that may land on a freed one's address
        q, _ = np.linalg.qr(np.random.default_rng(seed).standard_normal((128, 128)))
        fresh = torch.from_numpy(q.astype(np.float32)).to(dev)
        run(fresh)
        del fresh


def test_fused_encode_and_store_follows_changes_of_the_cache_object(golden, dev):
    """The function keeps what it has derived from a cache object per layer; everything that may change
    behind it -- cache tensors replaced or given other storage in place, the quantizer's matrix or boundaries
    replaced or rewritten in place, the block limit, the step's dtype / shape / slot dtype -- must be seen on the
    next call.  Every state is compared with fused_kv_update_pair on the same inputs."""
    class Cache:
        pass
    c = Cache()
    c.tq = make_tq(golden, dev, 4)
    c.block_size, c.max_blocks = 16, 6
    L, NB, H = 2, 6, 2
    c.k_packed = torch.zeros(L, NB, 16, H, 64, dtype=torch.uint8, device=dev)
    c.v_packed = torch.zeros_like(c.k_packed)
    c.k_norms = torch.zeros(L, NB, 16, H, device=dev)
    c.v_norms = torch.zeros_like(c.k_norms)
    g = torch.Generator(device=dev).manual_seed(3)

    def step(layer, tokens=9, dtype=torch.float16, slot_dtype=torch.int64):
        k = torch.randn(tokens, H, 128, device=dev, generator=g).to(dtype)
        v = torch.randn(tokens, H, 128, device=dev, generator=g).to(dtype)
        slots = (torch.randperm(NB * 16 + 8, device=dev, generator=g)[:tokens] - 4).to(slot_dtype)
        akv.fused_encode_and_store(c, layer, k, v, slots)
        want = [torch.zeros_like(x[layer]) for x in (c.k_packed, c.k_norms, c.v_packed, c.v_norms)]
        akv.fused_kv_update_pair(k, v, slots, want[0], want[1], want[2], want[3], c.tq.rotation, c.tq.boundaries_inner,
                                 c.tq.bits, block_size=c.block_size, max_blocks=c.max_blocks)
        written = want[1] != 0
        for got, w in zip((c.k_packed, c.k_norms, c.v_packed, c.v_norms), want):
            assert torch.equal(got[layer][written], w[written])
        return int(written.sum())

    assert step(0) > 0 and step(1) > 0 and step(0) > 0
    step(0, dtype=torch.bfloat16)
    step(0, dtype=torch.float32, slot_dtype=torch.int32)
    step(1, tokens=1)
    c.max_blocks = 3                                           # fewer blocks may be written
    c.k_norms.zero_(); c.v_norms.zero_()
    step(0, tokens=40)
    assert torch.all(c.k_norms[0, 3:] == 0)
    c.max_blocks = 6
    c.k_packed = torch.zeros_like(c.k_packed)                  # another tensor object
    c.k_norms = torch.zeros_like(c.k_norms)
    step(0)
    c.v_packed.set_(torch.zeros_like(c.v_packed))              # the same object over other storage
    step(0)
    c.tq.boundaries_inner.mul_(0.5)                            # rewritten in place
    step(1)
    c.tq.boundaries_inner = c.tq.boundaries_inner * 2.0        # replaced
    step(1)
    c.tq.rotation = c.tq.rotation.flip(0).contiguous()         # another matrix
    step(0)
    c.tq.rotation.copy_(torch.from_numpy(golden["rotation_d128_seed42"]).to(dev))
    step(0)
    c.k_packed = [c.k_packed[i].clone() for i in range(L)]     # a list of per-layer tensors, as the serving cache keeps them
    c.k_norms = [c.k_norms[i].clone() for i in range(L)]
    step(0)
    step(1)
    c.k_packed[0] = torch.zeros_like(c.k_packed[0])            # one element replaced inside the same list
    step(0)
    c.k_norms[1].data = torch.zeros_like(c.k_norms[1])         # an element given other storage
    step(1)
    c.v_norms.data = torch.zeros_like(c.v_norms)
    step(1)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tokens", [1, 37, 256])
def test_k_and_v_in_one_launch_equal_two_launches(golden, dev, bits, dtype, tokens):
    """fused_kv_update_pair against two fused_kv_update calls (those are checked against the oracle
    above): byte-identical caches and norms.  Token counts that leave the K / V seam inside a step of the
    kernel, padding slots, slots beyond max_blocks, and the K / V halves of one serving cache tensor
    (rows 4 bytes longer than the codes)."""
    tq = make_tq(golden, dev, bits)
    H, NB, BS, P = 8, 40, 16, tq._packed_dim
    g = torch.Generator(device=dev).manual_seed(1000 * bits + tokens)
    k = (torch.randn(tokens, H, 128, device=dev, generator=g) * 3).to(dtype)
    v = torch.randn(tokens, H, 128, device=dev, generator=g).to(dtype)
    slots = torch.randperm(NB * BS + 64, device=dev, generator=g)[:tokens] - 32        # some negative, some too large
    kv_a = torch.zeros(NB, 2, BS, H, P + 4, dtype=torch.uint8, device=dev)
    kv_b = torch.zeros_like(kv_a)
    norms_a = torch.zeros(2, NB, BS, H, device=dev)
    norms_b = torch.zeros_like(norms_a)
    akv.fused_kv_update_pair(k, v, slots, kv_a[:, 0], norms_a[0], kv_a[:, 1], norms_a[1], tq.rotation,
                             tq.boundaries_inner, bits, block_size=BS, max_blocks=NB - 1)
    akv.fused_kv_update(k, slots, kv_b[:, 0], norms_b[0], tq.rotation, tq.boundaries_inner, bits, BS, NB - 1)
    akv.fused_kv_update(v, slots, kv_b[:, 1], norms_b[1], tq.rotation, tq.boundaries_inner, bits, BS, NB - 1)
    assert torch.equal(kv_a, kv_b) and torch.equal(norms_a, norms_b)
    ok = (slots >= 0) & (slots < (NB - 1) * BS)
    assert int((norms_a[0] > 0).sum()) == int(ok.sum()) * H and torch.all(kv_a[..., P:] == 0)


def test_config1_literal_shape_steps_vs_oracle(golden, dev):
    """The serving write at its benchmark shape: 8 kv heads, a cache of 8,192 blocks of 16, steps of 256
    tokens (K and V) whose slots are consecutive runs of ONE random permutation of all 131,072 slots, so
    no step overwrites another.  After four steps the whole cache equals what the oracle's kv_update
    wrote: the same slots and nothing else, codes under the boundary-ulp rule, norms to 1e-6."""
    NB, BS, H, T, STEPS = 8192, 16, 8, 256, 4

    class Cache:
        pass
    c = Cache()
    c.tq = make_tq(golden, dev, 4)
    c.block_size, c.max_blocks = BS, NB
    c.k_packed = torch.zeros(1, NB, BS, H, 64, dtype=torch.uint8, device=dev)
    c.v_packed = torch.zeros_like(c.k_packed)
    c.k_norms = torch.zeros(1, NB, BS, H, device=dev)
    c.v_norms = torch.zeros_like(c.k_norms)
    rng = np.random.default_rng(1)
    perm = rng.permutation(NB * BS)
    R = golden["rotation_d128_seed42"]
    _, bnd, _ = O.get_codebook(128, 4)
    ref = {n: (np.zeros((NB, BS, H, 64), np.uint8), np.zeros((NB, BS, H), np.float32)) for n in "kv"}
    rows = {"k": [], "v": []}
    for step in range(STEPS):
        slots = perm[step * T:(step + 1) * T].astype(np.int64)
        k, v = kv_like(rng, (T, H, 128)), kv_like(rng, (T, H, 128))
        akv.fused_encode_and_store(c, 0, torch.from_numpy(k).to(dev), torch.from_numpy(v).to(dev),
                                   torch.from_numpy(slots).to(dev))
        for n, x in (("k", k), ("v", v)):
            O.kv_update(x, slots, ref[n][0], ref[n][1], R, bnd, block_size=BS, bits=4)
            rows[n].append((slots, x))
    for n, packed, norms in (("k", c.k_packed, c.k_norms), ("v", c.v_packed, c.v_norms)):
        got_p, got_n = packed[0].cpu().numpy(), norms[0].cpu().numpy()
        written = ref[n][1] > 0
        assert int(written.sum()) == STEPS * T * H and np.array_equal(got_n > 0, written)
        assert not got_p[~written].any()
        slots = np.concatenate([s for s, _ in rows[n]])
        x = np.concatenate([x for _, x in rows[n]])[np.argsort(slots)]             # rows in slot order, like the cache
        check_codes(got_p[written], got_n[written], x.reshape(-1, 128), R, 4, ref[n][0][written], ref[n][1][written])


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("n", [1, 33, 4097])
def test_decode_random_codes_vs_oracle(golden, dev, bits, n):
    """Every byte value occurs: the code spreading and the table lookups of the matrix-core decode."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(100 * bits + n)
    packed = rng.integers(0, 256, (n, tq._packed_dim), dtype=np.uint8)
    norms = rng.lognormal(1.0, 1.0, n).astype(np.float32)
    c, _, _ = O.get_codebook(128, bits)
    ref = O.decode(packed, norms, golden["rotation_d128_seed42"], c, bits).astype(np.float32)
    got = tq.decode(torch.from_numpy(packed).to(dev), torch.from_numpy(norms).to(dev)).cpu().numpy().astype(np.float32)
    tol = 2e-3 + np.abs(ref) * 2.0 ** -11          # half a float16 ulp of the output
    assert np.all(np.abs(got - ref) <= tol)
    assert np.mean(got == ref) > 0.99


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_decode_other_output_dtypes_vs_oracle(golden, dev, bits, dtype):
    tq = akv.TurboQuant(head_dim=128, bits=bits, device=str(dev), dtype=dtype)
    tq.rotation = torch.from_numpy(golden["rotation_d128_seed42"]).to(dev)
    rng = np.random.default_rng(7 * bits)
    n = 1031
    packed = rng.integers(0, 256, (n, tq._packed_dim), dtype=np.uint8)
    norms = rng.lognormal(1.0, 1.0, n).astype(np.float32)
    c, _, _ = O.get_codebook(128, bits)
    ref = O.decode(packed, norms, golden["rotation_d128_seed42"], c, bits, out_dtype=np.float32)
    out = tq.decode(torch.from_numpy(packed).to(dev), torch.from_numpy(norms).to(dev))
    assert out.dtype == dtype
    got = out.float().cpu().numpy()
    scale = np.abs(ref).max(axis=1, keepdims=True)
    if dtype == torch.float32:
        assert np.all(np.abs(got - ref) <= 4e-6 * scale + 1e-7)       # float32 sums in another order
    else:
        assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -8 + 4e-6 * scale)   # half a bfloat16 ulp


@pytest.mark.parametrize("bits,out_dtype,extra", [(4, torch.float16, 0), (4, torch.float16, 16), (4, torch.bfloat16, 0),
                                                  (3, torch.float16, 0), (2, torch.float32, 4),
                                                  (4, torch.float16, 4), (3, torch.bfloat16, 4)])
@pytest.mark.parametrize("itype", [torch.int32, torch.int64])
def test_batch_decompress_active_blocks_vs_oracle(golden, dev, bits, out_dtype, extra, itype):
    from aitherkvcache_amd.vllm import batch_decompress_active_blocks
    tq = make_tq(golden, dev, bits)
    R = golden["rotation_d128_seed42"]
    c, b, _ = O.get_codebook(128, bits)
    rng = np.random.default_rng(bits * 10 + extra)
    B, bs, H, pd = 23, 16, 3, tq._packed_dim
    caches, norms = [], []
    for _ in range(2):
        p, n = O.encode(kv_like(rng, (B, bs, H, 128)), R, b, bits)
        caches.append(np.concatenate([p, rng.integers(0, 256, (B, bs, H, extra), dtype=np.uint8)], axis=-1))
        norms.append(n)
    table = np.full((5, 6), -1, dtype=np.int64)
    table[0, :3] = [4, 9, 2]
    table[1, :6] = [9, 21, 22, 0, 17, 30]          # 9 shared; 21, 22 and 30 are outside num_blocks
    table[3, :1] = [20]
    num_blocks = 21
    ref = [np.full((B, bs, H, 128), 3.0, dtype=np.float32) for _ in range(2)]
    for i in range(2):
        O.batch_decompress_active_blocks(caches[i], norms[i], ref[i], table, num_blocks, R, c, bits, pd)
    bufs = [torch.full((B, bs, H, 128), 3.0, dtype=out_dtype, device=dev) for _ in range(2)]
    batch_decompress_active_blocks(
        torch.from_numpy(caches[0]).to(dev), torch.from_numpy(caches[1]).to(dev), bufs[0], bufs[1], tq, pd,
        torch.from_numpy(table).to(dev).to(itype), num_blocks,
        torch.from_numpy(norms[0]).to(dev), torch.from_numpy(norms[1]).to(dev))
    touched = np.zeros(B, dtype=bool)
    touched[[0, 2, 4, 9, 17, 20]] = True
    for i in range(2):
        got = bufs[i].float().cpu().numpy()
        assert np.all(got[~touched] == 3.0)                       # unlisted blocks untouched
        # the oracle rounds to float16 as tq.decode does: allow half an ulp of the coarser of the two formats
        rel = {torch.float16: 0.0, torch.bfloat16: 2.0 ** -8, torch.float32: 2.0 ** -11}[out_dtype]
        tol = 2e-3 + np.abs(ref[i][touched]) * rel
        assert np.all(np.abs(got[touched] - ref[i][touched]) <= tol)
        if out_dtype == torch.float16:
            assert np.mean(got[touched] == ref[i][touched]) > 0.995


def test_batch_decompress_empty_and_errors(golden, dev):
    from aitherkvcache_amd.vllm import decode_blocks
    tq = make_tq(golden, dev, 4)
    cache = torch.zeros(4, 16, 2, 64, dtype=torch.uint8, device=dev)
    norms = torch.ones(4, 16, 2, device=dev)
    buf = torch.full((4, 16, 2, 128), 5.0, dtype=torch.float16, device=dev)
    decode_blocks(cache, norms, buf, tq, torch.empty(0, dtype=torch.int64, device=dev), 4)
    decode_blocks(cache, norms, buf, tq, torch.tensor([-1, 7], device=dev), 4)
    assert torch.all(buf == 5.0)
    with pytest.raises(ValueError):
        decode_blocks(cache, norms, buf, tq, torch.tensor([0], device=dev), 5)
    with pytest.raises(ValueError):
        decode_blocks(cache[..., :32], norms, buf, tq, torch.tensor([0], device=dev), 4)
    with pytest.raises(RuntimeError):
        decode_blocks(cache.cpu(), norms.cpu(), buf.cpu(), tq, torch.tensor([0]), 4)


def test_config0_round_trip_full_size(golden, dev):
    """65,536 x 128 fp16, 4-bit: every code accounted for, distortion at the table value."""
    tq = make_tq(golden, dev, 4)
    rng = np.random.default_rng(0)
    x = kv_like(rng, (65536, 128))
    xt = torch.from_numpy(x).to(dev)
    packed, norms = tq.encode(xt)
    n = check_codes(packed.cpu().numpy(), norms.cpu().numpy(), x, golden["rotation_d128_seed42"], 4)
    print(f"[config0] mismatching codes: {n} of {65536 * 128}")
    xh = tq.decode(packed, norms).float()
    xf = xt.float()
    rel = ((xf - xh).pow(2).sum(-1) / xf.pow(2).sum(-1)).mean().item()
    assert abs(rel - 0.0095) / 0.0095 < 0.05
    # idempotence: re-encoding the reconstruction reproduces the codes (same cell) almost everywhere
    p2, _ = tq.encode(xh)
    assert (p2 == packed).float().mean().item() > 0.97
    rep = tq.validate(num_vectors=20000)
    assert rep["mse_theory_lower"] <= rep["mse"] <= rep["mse_theory_upper"] and rep["hip_active"]


def test_gpu_cache_encode_spill_warm(golden, dev):
    """TQGPUCache (reference: vllm/cache.py:22-173): encode_and_store equals the fused update on the
    layer's tensors, spilled blocks survive being overwritten on the device and come back bit for
    bit, blocks that were never spilled are left alone by warm_blocks."""
    from aitherkvcache_amd.vllm import TQGPUCache

    def t(a, dev):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    cache = TQGPUCache(num_layers=3, max_blocks=24, block_size=16, num_kv_heads=4, head_dim=128, bits=4, device=str(dev))
    cache.tq.rotation = torch.from_numpy(golden["rotation_d128_seed42"]).to(dev)
    rng = np.random.default_rng(77)
    T = 150
    slots = rng.permutation(24 * 16)[:T].astype(np.int64)
    slots[5] = -1                                             # a padding token
    for layer in range(3):
        key, val = kv_like(rng, (T, 4, 128)), kv_like(rng, (T, 4, 128))
        cache.encode_and_store(layer, t(key, dev), t(val, dev), t(slots, dev))
        kp = torch.zeros_like(cache.k_packed[layer]); kn = torch.zeros_like(cache.k_norms[layer])
        akv.fused_tq4_kv_update(t(key, dev), t(slots, dev), kp, kn, cache.tq.rotation, cache.tq.boundaries_inner)
        assert torch.equal(kp, cache.k_packed[layer]) and torch.equal(kn, cache.k_norms[layer])
        assert int(cache.v_norms[layer].count_nonzero()) == (T - 1) * 4
    snap = [x.clone() for x in (cache._k_packed, cache._k_norms, cache._v_packed, cache._v_norms)]
    spill = torch.tensor([3, 17, 0, 9], device=dev)
    cache.spill_blocks(spill)
    assert cache.has_spilled(17) and not cache.has_spilled(4)
    stats = cache.cold_tier_stats()
    assert stats["cold_blocks"] == 4 and stats["cold_tokens"] == 64 and stats["max_blocks"] == 24
    assert abs(stats["cold_mb"] - 4 * 2 * 16 * 4 * 68 * 3 / 2 ** 20) < 1e-9
    for x in (cache._k_packed, cache._k_norms, cache._v_packed, cache._v_norms):
        x[:, spill] = 0                                       # the device blocks are reused
        x[:, 5] = 0                                           # so is one that was never spilled
    cache.warm_blocks(torch.tensor([17, 5, 3, 0, 9]))
    torch.cuda.synchronize()
    for now, before in zip((cache._k_packed, cache._k_norms, cache._v_packed, cache._v_norms), snap):
        keep = torch.ones(24, dtype=torch.bool, device=dev)
        keep[5] = False
        assert torch.equal(now[:, keep], before[:, keep])
        assert not bool(now[:, 5].any())
    cache.clear_spilled([3, 9])
    assert not cache.has_spilled(3) and cache.has_spilled(0)
    cache.spill_blocks(torch.empty(0, dtype=torch.long))
    cache.warm_blocks(torch.empty(0, dtype=torch.long))


def test_read_probe_sums_what_it_reads(dev):
    """The read probe of the benchmarks: every 16-byte piece is read exactly once (the folded sum of the words
    of a known buffer comes out), sizes that are no multiple of the unrolled step included."""
    L = _lib.lib()
    for n16 in (1, 255, 4096 * 37 + 5):
        words = torch.arange(4 * n16, dtype=torch.int64, device=dev) % 251
        buf = words.to(torch.int32).contiguous()
        sink = torch.zeros(64, dtype=torch.int32, device=dev)
        _lib.check(L.akv_debug_read_probe(buf.data_ptr(), 16 * n16, sink.data_ptr(), _lib.stream_ptr(dev)))
        w = words.view(n16, 4)
        per_piece = (w[:, 0] ^ w[:, 1]) + (w[:, 2] ^ w[:, 3])
        # a lane folds its 32-bit sum to 16 bits before the wavefront adds up in float32; small values keep that exact
        assert int(sink.sum().item()) == int(per_piece.sum().item())
    with pytest.raises(ValueError):
        _lib.check(L.akv_debug_read_probe(0, 16, sink.data_ptr(), _lib.stream_ptr(dev)))


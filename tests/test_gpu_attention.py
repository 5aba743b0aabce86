"""Paged decode attention over the TurboQuant cache (HIP, through the C ABI) against the
reference's own outputs and the oracle.  Tolerance: 2e-3 max-abs on fp16 outputs."""
import math

import numpy as np
import pytest
import torch

import aitherkvcache_amd as akv
from oracle import tq_oracle as O
from tests.util import kv_like

pytestmark = pytest.mark.gpu
TOL = 2e-3


def within_tol(got, ref64):
    """|got - ref| <= 2e-3, plus the rounding of the fp16 output itself (half an fp16 ulp =
    2**-11 relative) where |ref| is large enough for that to matter (|out| >= 4)."""
    got = np.asarray(got, dtype=np.float64)
    return bool(np.all(np.abs(got - ref64) <= TOL + 2.0 ** -11 * np.abs(ref64)))


def make_tq(golden, dev, bits):
    tq = akv.TurboQuant(head_dim=128, bits=bits, device=str(dev))
    tq.rotation = torch.from_numpy(golden["rotation_d128_seed42"]).to(dev)
    return tq


def t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("itype", [torch.int64, torch.int32])
def test_golden_outputs(golden, dev, bits, itype):
    tq = make_tq(golden, dev, bits)
    attn = akv.TQPagedAttention(tq, num_query_heads=8)
    tables = golden["attn_tables"]          # holds a 10**6 padding entry that must never be read
    out = attn.forward(t(golden["attn_q"], dev), t(golden[f"attn_kp_b{bits}"], dev),
                       t(golden[f"attn_kn_b{bits}"], dev), t(golden[f"attn_vp_b{bits}"], dev),
                       t(golden[f"attn_vn_b{bits}"], dev), t(tables, dev).to(itype),
                       t(golden["attn_ctx"], dev).to(itype), block_size=16, num_kv_heads=2)
    assert out.dtype == torch.float16 and out.shape == (4, 8, 128)
    got = out.cpu().numpy().astype(np.float32)
    ref = golden[f"attn_out_b{bits}"].astype(np.float32)
    assert np.all(got[0] == 0)                                   # ctx == 0 -> zeros
    err = np.max(np.abs(got - ref))
    print(f"[attn golden] bits={bits} max|diff|={err:.2e} exact={np.mean(got == ref):.4f}")
    assert err <= TOL


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_reference_named_class_golden_outputs(golden, dev, bits):
    """TQPagedAttentionRef takes the rotation, the codebook and the scale as the reference's class of that name
    does; its results are the reference's golden outputs."""
    from aitherkvcache_amd.fused_attention import TQPagedAttentionRef
    tq = make_tq(golden, dev, bits)
    ref_attn = TQPagedAttentionRef(tq.rotation, tq.centroids, 1.0 / math.sqrt(128), num_kv_heads=2, num_query_heads=8,
                                   head_dim=128, block_size=16, bits=bits)
    out = ref_attn.forward(t(golden["attn_q"], dev), t(golden[f"attn_kp_b{bits}"], dev),
                           t(golden[f"attn_kn_b{bits}"], dev), t(golden[f"attn_vp_b{bits}"], dev),
                           t(golden[f"attn_vn_b{bits}"], dev), t(golden["attn_tables"], dev), t(golden["attn_ctx"], dev))
    got = out.cpu().numpy().astype(np.float32)
    assert np.max(np.abs(got - golden[f"attn_out_b{bits}"].astype(np.float32))) <= TOL
    # the scale is the caller's: twice the scale is not the same attention
    other = TQPagedAttentionRef(tq.rotation, tq.centroids, 2.0 / math.sqrt(128), 2, 8, 128, 16, bits)
    out2 = other.forward(t(golden["attn_q"], dev), t(golden[f"attn_kp_b{bits}"], dev),
                         t(golden[f"attn_kn_b{bits}"], dev), t(golden[f"attn_vp_b{bits}"], dev),
                         t(golden[f"attn_vn_b{bits}"], dev), t(golden["attn_tables"], dev), t(golden["attn_ctx"], dev))
    assert float((out2.float() - out.float()).abs().max()) > 1e-2


def build_cache(rng, tq, dev, num_blocks, kvh, bits, block_size=16, pad=0):
    """Random K/V written through the HIP encode-on-write kernel.  Returns device tensors and the
    host copies the oracle reads."""
    P = tq._packed_dim
    T = num_blocks * block_size
    keys = kv_like(rng, (T, kvh, 128))
    vals = kv_like(rng, (T, kvh, 128))
    kp = torch.zeros(num_blocks, block_size, kvh, P + pad, dtype=torch.uint8, device=dev)
    vp = torch.zeros_like(kp)
    kn = torch.zeros(num_blocks, block_size, kvh, device=dev)
    vn = torch.zeros_like(kn)
    slots = torch.arange(T, device=dev)
    akv.fused_kv_update(t(keys, dev), slots, kp, kn, tq.rotation, tq.boundaries_inner, bits, block_size)
    akv.fused_kv_update(t(vals, dev), slots, vp, vn, tq.rotation, tq.boundaries_inner, bits, block_size)
    return kp, kn, vp, vn


def oracle_rows_of_batch(q, kp, kn, vp, vn, tables, ctx, golden, bits, seqs, block_size=16):
    """Float64 oracle outputs for the sequences `seqs` of a batch, one sequence at a time (bounded memory);
    the cache tensors are brought to the host once."""
    c, _, _ = O.get_codebook(128, bits)
    host = [x.cpu().numpy() for x in (kp, kn, vp, vn)]
    R = golden["rotation_d128_seed42"]
    return {s: O.paged_attention(q[s:s + 1], host[0], host[1], host[2], host[3], tables[s:s + 1], ctx[s:s + 1], R, c,
                                 bits, block_size=block_size, dtype=np.float64, cast_output=False)[0] for s in seqs}


def oracle_out(q, kp, kn, vp, vn, tables, ctx, golden, bits, block_size=16, P=None):
    c, _, _ = O.get_codebook(128, bits)
    P = P or kp.shape[-1]
    return O.paged_attention(q, kp.cpu().numpy()[..., :P], kn.cpu().numpy(), vp.cpu().numpy()[..., :P],
                             vn.cpu().numpy(), tables, ctx, golden["rotation_d128_seed42"], c, bits,
                             block_size=block_size, dtype=np.float64, cast_output=False)


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("qh,kvh", [(32, 8), (8, 8), (6, 2), (16, 2), (32, 2), (24, 2), (9, 1), (40, 2), (16, 16), (24, 12), (48, 6)])
def test_ragged_batch_vs_oracle(golden, dev, bits, qh, kvh):
    """Ragged contexts (0, 1, partial block, many blocks), permuted non-contiguous tables, GQA
    ratios 4 / 1 / 3 / 8, and 16 / 12 / 9 / 20 (a kv head presented as two or three groups of query
    heads on the matrix-core kernel); 16 and 12 kv heads, and 6 kv heads as 12 groups, take two passes of
    eight head slots on that kernel, the second with eight or four active slots."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(200 + bits + qh)
    NB = 96
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, kvh, bits)
    ctx = np.array([0, 1, 15, 16, 17, 333, 700, 64], dtype=np.int64)
    width = 48
    tables = np.full((len(ctx), width), -7, dtype=np.int64)             # garbage padding
    for s, c_ in enumerate(ctx):
        nb = -(-int(c_) // 16)
        tables[s, :nb] = rng.permutation(NB)[:nb]
    q = rng.standard_normal((len(ctx), qh, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, num_query_heads=qh)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), block_size=16, num_kv_heads=kvh)
    ref = oracle_out(q, kp, kn, vp, vn, tables, ctx, golden, bits)
    got = out.cpu().numpy().astype(np.float64)
    err = np.max(np.abs(got - ref))
    print(f"[attn ragged] bits={bits} qh={qh} kvh={kvh} max|diff|={err:.2e} max|out|={np.abs(ref).max():.2f}")
    assert np.all(got[0] == 0)
    assert within_tol(got, ref)
    # float32 queries give float32 outputs, closer still
    out32 = attn.forward(t(q.astype(np.float32), dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), 16, kvh)
    assert out32.dtype == torch.float32
    # float32 in/out isolates the arithmetic: the general kernels are float32 throughout (~1e-6);
    # the MFMA kernel's fp16 codebook table costs ~1e-4 relative, i.e. up to ~6e-4 at |out| ~ 5
    assert np.max(np.abs(out32.cpu().numpy() - ref)) <= 1e-3


@pytest.mark.parametrize("bits", [4, 3])
def test_batch_of_many_sequences_vs_oracle(golden, dev, bits):
    """330 sequences of 0..90 tokens x 32 query heads: more (sequence, kv head) and (sequence, four heads) items
    than the rotation blocks of the prologue and the workgroups of the reduce kernel, which then take several
    items each; more than 63 sequences also take the scalar search for a segment's sequence."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(900 + bits)
    NB, S, qh, kvh = 64, 330, 32, 8
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, kvh, bits)
    ctx = rng.integers(0, 91, size=S).astype(np.int64)
    ctx[:4] = [0, 1, 16, 90]
    width = 8
    tables = np.full((S, width), -3, dtype=np.int64)
    for s_, c_ in enumerate(ctx):
        nb = -(-int(c_) // 16)
        tables[s_, :nb] = rng.permutation(NB)[:nb]
    q = rng.standard_normal((S, qh, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, num_query_heads=qh)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), block_size=16, num_kv_heads=kvh)
    ref = oracle_out(q, kp, kn, vp, vn, tables, ctx, golden, bits)
    got = out.cpu().numpy().astype(np.float64)
    print(f"[attn many sequences] bits={bits} max|diff|={np.max(np.abs(got - ref)):.2e}")
    assert np.all(got[0] == 0)
    assert within_tol(got, ref)
    out32 = attn.forward(t(q.astype(np.float32), dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), 16, kvh)
    assert np.max(np.abs(out32.cpu().numpy() - ref)) <= 1e-3


def test_serving_layout_strided_views(golden, dev):
    """K/V as views of one uint8 [blocks, 2, bs, heads, 68] tensor (row pitch 68 bytes) and norms
    as a slice of a [layers, blocks, bs, heads] tensor."""
    tq = make_tq(golden, dev, 4)
    rng = np.random.default_rng(31)
    NB, BS, KVH, QH = 40, 16, 8, 32
    cache = torch.zeros(NB, 2, BS, KVH, 68, dtype=torch.uint8, device=dev)
    norms = torch.zeros(2, 3, NB, BS, KVH, device=dev)
    T = NB * BS
    keys, vals = kv_like(rng, (T, KVH, 128)), kv_like(rng, (T, KVH, 128))
    slots = torch.arange(T, device=dev)
    akv.fused_tq4_kv_update(t(keys, dev), slots, cache[:, 0], norms[0, 1], tq.rotation, tq.boundaries_inner)
    akv.fused_tq4_kv_update(t(vals, dev), slots, cache[:, 1], norms[1, 1], tq.rotation, tq.boundaries_inner)
    ctx = np.array([640, 100, 37], dtype=np.int32)
    tables = np.stack([rng.permutation(NB) for _ in range(3)]).astype(np.int32)
    q = rng.standard_normal((3, QH, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, QH)
    out = attn.forward(t(q, dev), cache[:, 0][..., :64], norms[0, 1], cache[:, 1][..., :64], norms[1, 1],
                       t(tables, dev), t(ctx, dev))
    ref = oracle_out(q, cache[:, 0], norms[0, 1], cache[:, 1], norms[1, 1], tables, ctx, golden, 4, P=64)
    assert within_tol(out.cpu().numpy(), ref)


@pytest.mark.parametrize("block_size", [8, 32])
def test_other_block_sizes(golden, dev, block_size):
    tq = make_tq(golden, dev, 4)
    rng = np.random.default_rng(block_size)
    NB, KVH, QH = 24, 2, 8
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, KVH, 4, block_size=block_size)
    ctx = np.array([block_size * 5 + 3, 2], dtype=np.int64)
    tables = np.stack([rng.permutation(NB)[:8] for _ in range(2)])
    q = rng.standard_normal((2, QH, 128)).astype(np.float16)
    out = akv.TQPagedAttention(tq, QH).forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev),
                                               block_size=block_size)
    ref = oracle_out(q, kp, kn, vp, vn, tables, ctx, golden, 4, block_size=block_size)
    assert within_tol(out.cpu().numpy(), ref)


@pytest.mark.parametrize("bits", [4, 3, 2])
def test_blocks_of_32_tokens(golden, dev, bits):
    """Blocks of 32 tokens (one chunk of the matrix-core kernel = one block, its second 16-token tile
    sixteen positions in): ragged batch against the oracle, then a batch large enough that every
    workgroup runs through several windows of block ids, checked by the uniform-value property and,
    for one sequence, against the oracle."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(320 + bits)
    KVH, QH, BS = 8, 32, 32
    NB = 200
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, KVH, bits, block_size=BS)
    ctx = np.array([1, 31, 32, 33, 1000, 0, 2048, 777], dtype=np.int64)
    tables = np.full((len(ctx), 64), -5, dtype=np.int64)
    perm = rng.permutation(NB)
    off = 0
    for s_, c_ in enumerate(ctx):
        nb = -(-int(c_) // BS)
        tables[s_, :nb] = perm[off:off + nb]
        off += nb
    q = rng.standard_normal((len(ctx), QH, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, QH)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), block_size=BS)
    ref = oracle_out(q, kp, kn, vp, vn, np.maximum(tables, 0), ctx, golden, bits, block_size=BS)
    assert within_tol(out.cpu().numpy(), ref) and not bool(out[5].any())
    # large: 16 sequences x 32768 tokens
    S, CTX = 16, 32768
    nb_seq = CTX // BS
    NBL = S * nb_seq
    P = tq._packed_dim
    kpl = torch.empty(NBL, BS, KVH, P, dtype=torch.uint8, device=dev)
    knl = torch.empty(NBL, BS, KVH, device=dev)
    gen = torch.Generator(device=dev).manual_seed(11)
    CH = 1024
    for b0 in range(0, NBL, CH):
        b1 = min(NBL, b0 + CH)
        x = torch.randn((b1 - b0) * BS * KVH, 128, device=dev, generator=gen).half()
        pk, nr = tq.encode(x)
        kpl[b0:b1] = pk.reshape(b1 - b0, BS, KVH, P)
        knl[b0:b1] = nr.reshape(b1 - b0, BS, KVH)
    v1 = kv_like(rng, (1, KVH, 128))
    vp1, vn1 = tq.encode(t(v1, dev))
    vpl = vp1.reshape(1, 1, KVH, P).expand(NBL, BS, KVH, P).contiguous()
    vnl = vn1.reshape(1, 1, KVH).expand(NBL, BS, KVH).contiguous()
    tabl = rng.permutation(NBL).reshape(S, nb_seq).astype(np.int32)
    ctxl = np.full(S, CTX, dtype=np.int64)
    ctxl[3], ctxl[9] = CTX - 45, 3000
    ql = rng.standard_normal((S, QH, 128)).astype(np.float16)
    outl = attn.forward(t(ql, dev), kpl, knl, vpl, vnl, t(tabl, dev), t(ctxl, dev), block_size=BS).float()
    want = tq.decode(vp1, vn1).float().reshape(KVH, 1, 128).expand(KVH, 4, 128).reshape(1, QH, 128)
    assert bool(torch.all(torch.abs(outl - want) <= TOL + 2.0 ** -10 * want.abs()))
    s_ = 9
    vp_r, vn_r = kpl.roll(3, 0), knl.roll(3, 0)
    o = attn.forward(t(ql[s_:s_ + 1], dev), kpl, knl, vp_r, vn_r, t(tabl[s_:s_ + 1], dev), t(ctxl[s_:s_ + 1], dev),
                     block_size=BS)
    nbu = -(-int(ctxl[s_]) // BS)
    used = np.unique(tabl[s_, :nbu])
    remap = {b: i for i, b in enumerate(used)}
    small_tab = np.array([[remap[b] for b in tabl[s_, :nbu]]])
    idx = t(used.astype(np.int64), dev)
    ref1 = oracle_out(ql[s_:s_ + 1], kpl[idx], knl[idx], vp_r[idx], vn_r[idx], small_tab, ctxl[s_:s_ + 1], golden, bits,
                      block_size=BS)
    assert within_tol(o.cpu().numpy(), ref1)


def test_long_context_split_invariants(golden, dev):
    """Sizes where a sequence is cut across many workgroups: results must not depend on where the
    cuts fall.  (a) against the float64 oracle; (b) the same sequence alone or inside a batch
    that shifts every cut; (c) a block-table permutation with the blocks moved accordingly."""
    tq = make_tq(golden, dev, 4)
    rng = np.random.default_rng(99)
    NB, KVH, QH = 1600, 8, 32
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, KVH, 4)
    ctx = np.array([12000, 1030, 5000, 7531], dtype=np.int64)
    width = 800
    tables = np.zeros((4, width), dtype=np.int64)
    perm = rng.permutation(NB)
    off = 0
    for s, c_ in enumerate(ctx):
        nb = -(-int(c_) // 16)
        tables[s, :nb] = perm[off:off + nb]
        off += nb
    q = rng.standard_normal((4, QH, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, QH)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev)).cpu().numpy().astype(np.float64)
    ref = oracle_out(q, kp, kn, vp, vn, tables, ctx, golden, 4)
    err = np.max(np.abs(out - ref))
    print(f"[attn long] max|diff|={err:.2e}")
    assert within_tol(out, ref)
    # the invariance checks use float32 queries so that no fp16 output rounding blurs them
    q32 = t(q.astype(np.float32), dev)
    full = attn.forward(q32, kp, kn, vp, vn, t(tables, dev), t(ctx, dev)).cpu().numpy()
    assert np.max(np.abs(full - ref)) <= 1e-3
    solo = attn.forward(q32[2:3], kp, kn, vp, vn, t(tables[2:3], dev), t(ctx[2:3], dev)).cpu().numpy()
    assert np.max(np.abs(solo - full[2:3])) <= 2e-5
    # move every physical block and remap the tables
    mv = rng.permutation(NB)
    inv = np.argsort(mv)
    out2 = attn.forward(q32, kp[t(mv, dev)], kn[t(mv, dev)], vp[t(mv, dev)], vn[t(mv, dev)],
                        t(inv[tables], dev), t(ctx, dev)).cpu().numpy()
    assert np.max(np.abs(out2 - full)) <= 2e-5


def test_config2_shape_properties(golden, dev):
    """Llama-3-8B layer shape at benchmark scale (32Q/8KV, batch 16, ctx U[1k, 40k]): the softmax weights must
    sum to one (uniform values -> output equals the value), the shortest sequence run alone equals the oracle,
    and EVERY sequence of the full-batch launch with random values equals the oracle (a wrong table column or
    partial slot anywhere in the 16-sequence launch shows there)."""
    tq = make_tq(golden, dev, 4)
    rng = np.random.default_rng(2)
    ctx = rng.integers(1024, 40961, size=16).astype(np.int64)
    nblk = -(-ctx // 16)
    NB = int(nblk.sum())
    KVH, QH = 8, 32
    # K random; V = one fixed vector everywhere -> attention output must be that vector decoded
    kp = torch.zeros(NB, 16, KVH, 64, dtype=torch.uint8, device=dev)
    kn = torch.zeros(NB, 16, KVH, device=dev)
    gen = torch.Generator(device=dev).manual_seed(5)
    CH = 2048
    for b0 in range(0, NB, CH):
        b1 = min(NB, b0 + CH)
        x = torch.randn((b1 - b0) * 16, KVH, 128, device=dev, generator=gen).half()
        akv.fused_tq4_kv_update(x, torch.arange(b0 * 16, b1 * 16, device=dev), kp, kn, tq.rotation,
                                tq.boundaries_inner)
    v1 = kv_like(rng, (1, KVH, 128))
    vp1, vn1 = tq.encode(t(v1, dev))
    vp = vp1.reshape(1, 1, KVH, 64).expand(NB, 16, KVH, 64).contiguous()
    vn = vn1.reshape(1, 1, KVH).expand(NB, 16, KVH).contiguous()
    perm = rng.permutation(NB)
    tables = np.zeros((16, int(nblk.max())), dtype=np.int32)
    off = 0
    for s in range(16):
        tables[s, :nblk[s]] = perm[off:off + nblk[s]]
        off += nblk[s]
    q = rng.standard_normal((16, QH, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, QH)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev)).float()
    want = tq.decode(vp1, vn1).float().reshape(KVH, 1, 128).expand(KVH, 4, 128).reshape(1, QH, 128)
    # both sides are fp16-rounded: allow one fp16 ulp on top of the tolerance
    assert bool(torch.all(torch.abs(out - want) <= TOL + 2.0 ** -10 * want.abs()))
    # shortest sequence against the oracle with random V
    s = int(np.argmin(ctx))
    vp_r, vn_r = kp.roll(5, 0), kn.roll(5, 0)
    o = attn.forward(t(q[s:s + 1], dev), kp, kn, vp_r, vn_r, t(tables[s:s + 1], dev), t(ctx[s:s + 1], dev))
    used = np.unique(tables[s, :nblk[s]])
    remap = {b: i for i, b in enumerate(used)}
    small_tab = np.array([[remap[b] for b in tables[s, :nblk[s]]]])
    idx = t(used.astype(np.int64), dev)
    ref = oracle_out(q[s:s + 1], kp[idx], kn[idx], vp_r[idx], vn_r[idx], small_tab, ctx[s:s + 1], golden, 4)
    assert within_tol(o.cpu().numpy(), ref)
    # the whole batch in ONE launch, random values, every sequence against the oracle
    full = attn.forward(t(q, dev), kp, kn, vp_r, vn_r, t(tables, dev), t(ctx, dev)).cpu().numpy()
    full32 = attn.forward(t(q.astype(np.float32), dev), kp, kn, vp_r, vn_r, t(tables, dev), t(ctx, dev)).cpu().numpy()
    refs = oracle_rows_of_batch(q, kp, kn, vp_r, vn_r, tables, ctx, golden, 4, range(16))
    worst = 0.0
    for s_, r_ in refs.items():
        assert within_tol(full[s_], r_), f"sequence {s_} of the full batch"
        worst = max(worst, float(np.max(np.abs(full32[s_] - r_))))
    print(f"[attn config 2] all 16 sequences in one launch: float32 max|diff|={worst:.2e}")
    assert worst <= 1e-3


@pytest.mark.parametrize("bits", [3, 2])
def test_config3_shape_properties(golden, dev, bits):
    """The 3-bit and 2-bit benchmark shape (32Q/8KV, 64 sequences x 8192 tokens, block 16): (a) with one value
    row everywhere the output must be that row decoded, whatever the scores and wherever the workgroup cuts
    fall; (b) one whole sequence, run alone, with random values against the oracle; (c) the full batch in ONE
    launch with random values: ten sequences spread over the batch, the ragged and the one-token one among
    them, against the oracle."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(3)
    S, CTX, KVH, QH = 64, 8192, 8, 32
    nb_seq = CTX // 16
    NB = S * nb_seq
    P = tq._packed_dim
    kp = torch.empty(NB, 16, KVH, P, dtype=torch.uint8, device=dev)
    kn = torch.empty(NB, 16, KVH, device=dev)
    gen = torch.Generator(device=dev).manual_seed(7)
    CH = 2048
    for b0 in range(0, NB, CH):
        b1 = min(NB, b0 + CH)
        x = torch.randn((b1 - b0) * 16 * KVH, 128, device=dev, generator=gen).half()
        pk, nr = tq.encode(x)
        kp[b0:b1] = pk.reshape(b1 - b0, 16, KVH, P)
        kn[b0:b1] = nr.reshape(b1 - b0, 16, KVH)
    v1 = kv_like(rng, (1, KVH, 128))
    vp1, vn1 = tq.encode(t(v1, dev))
    vp = vp1.reshape(1, 1, KVH, P).expand(NB, 16, KVH, P).contiguous()
    vn = vn1.reshape(1, 1, KVH).expand(NB, 16, KVH).contiguous()
    tables = rng.permutation(NB).reshape(S, nb_seq).astype(np.int32)
    ctx = np.full(S, CTX, dtype=np.int64)
    ctx[5], ctx[17] = CTX - 9, 1          # a ragged end and a one-token sequence
    q = rng.standard_normal((S, QH, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, QH)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev)).float()
    want = tq.decode(vp1, vn1).float().reshape(KVH, 1, 128).expand(KVH, 4, 128).reshape(1, QH, 128)
    assert bool(torch.all(torch.abs(out - want) <= TOL + 2.0 ** -10 * want.abs()))
    s = 5
    vp_r, vn_r = kp.roll(3, 0), kn.roll(3, 0)
    o = attn.forward(t(q[s:s + 1], dev), kp, kn, vp_r, vn_r, t(tables[s:s + 1], dev), t(ctx[s:s + 1], dev))
    used = np.unique(tables[s])
    remap = {b: i for i, b in enumerate(used)}
    small_tab = np.array([[remap[b] for b in tables[s]]])
    idx = t(used.astype(np.int64), dev)
    ref = oracle_out(q[s:s + 1], kp[idx], kn[idx], vp_r[idx], vn_r[idx], small_tab, ctx[s:s + 1], golden, bits)
    err = np.max(np.abs(o.cpu().numpy().astype(np.float64) - ref))
    print(f"[attn config 3, {bits}-bit] one sequence max|diff|={err:.2e}")
    assert within_tol(o.cpu().numpy(), ref)
    full = attn.forward(t(q, dev), kp, kn, vp_r, vn_r, t(tables, dev), t(ctx, dev)).cpu().numpy()
    refs = oracle_rows_of_batch(q, kp, kn, vp_r, vn_r, tables, ctx, golden, bits, (0, 5, 6, 17, 18, 31, 32, 40, 57, 63))
    for s_, r_ in refs.items():
        assert within_tol(full[s_], r_), f"sequence {s_} of the full batch"


def test_decode_step_custom_op(golden, dev):
    """tq::decode_step: encode the step's token into the serving cache, attend, write output."""
    from aitherkvcache_amd.vllm import hooks
    hooks.reset_state()
    assert hooks.register_custom_ops()
    tq = hooks.init_quantizer(128, bits=4, device=str(dev))
    tq.rotation = torch.from_numpy(golden["rotation_d128_seed42"]).to(dev)
    rng = np.random.default_rng(55)
    NB, BS, KVH, QH, L = 12, 16, 2, 8, 2
    kv_cache = torch.zeros(NB, 2, BS, KVH, 68, dtype=torch.uint8, device=dev)
    k_norms = torch.zeros(L, NB, BS, KVH, device=dev)
    v_norms = torch.zeros_like(k_norms)
    hist = 37                                              # tokens already in the cache per sequence
    tables = np.stack([np.array([3, 7, 1, 0]), np.array([9, 2, 5, 0])]).astype(np.int32)
    keys, vals = kv_like(rng, (2, hist + 1, KVH, 128)), kv_like(rng, (2, hist + 1, KVH, 128))
    for s in range(2):
        slots = np.array([tables[s, p // BS] * BS + p % BS for p in range(hist)])
        akv.fused_tq4_kv_update(t(keys[s, :hist], dev), t(slots, dev), kv_cache[:, 0], k_norms[1], tq.rotation, tq.boundaries_inner)
        akv.fused_tq4_kv_update(t(vals[s, :hist], dev), t(slots, dev), kv_cache[:, 1], v_norms[1], tq.rotation, tq.boundaries_inner)
    new_slots = np.array([tables[s, hist // BS] * BS + hist % BS for s in range(2)] + [-1], dtype=np.int64)
    q = rng.standard_normal((3, QH, 128)).astype(np.float16)           # third row is padding
    key = np.concatenate([keys[:, hist], np.zeros((1, KVH, 128), np.float16)])
    val = np.concatenate([vals[:, hist], np.zeros((1, KVH, 128), np.float16)])
    output = torch.zeros(3, QH, 128, dtype=torch.float16, device=dev)
    seq_lens = np.array([hist + 1, hist + 1], dtype=np.int32)
    ret = torch.ops.tq.decode_step(t(q, dev), t(key, dev), t(val, dev), kv_cache, output, k_norms, v_norms,
                                   t(new_slots, dev), t(tables, dev), t(seq_lens, dev), 1, QH, KVH, 128,
                                   1 / math.sqrt(128), 2)
    assert torch.equal(ret, output) and torch.all(output[2] == 0)
    ref = oracle_out(q[:2], kv_cache[:, 0], k_norms[1], kv_cache[:, 1], v_norms[1], tables, seq_lens, golden, 4, P=64)
    assert within_tol(output[:2].cpu().numpy(), ref)
    # the new token really was written (its norm is in place), layer 0 untouched
    assert float(k_norms[1, tables[0, hist // BS], hist % BS, 0]) > 0 and torch.all(k_norms[0] == 0)


def test_decode_step_replays_from_a_graph(golden, dev):
    """The decode step (two encode-on-write launches and the attention launches) recorded into a HIP
    graph: every replay, with eager work and synchronisations in between and fresh inputs copied into
    the graph's static tensors, must equal the eager result for those inputs."""
    from aitherkvcache_amd.vllm import hooks
    hooks.reset_state()
    assert hooks.register_custom_ops()
    tq = hooks.init_quantizer(128, bits=4, device=str(dev))
    tq.rotation = torch.from_numpy(golden["rotation_d128_seed42"]).to(dev)
    rng = np.random.default_rng(56)
    NB, BS, KVH, QH, L, S = 400, 16, 8, 32, 1, 4
    hist = np.array([1500, 37, 640, 1023])
    tables = rng.permutation(NB)[:S * 96].reshape(S, 96).astype(np.int32)

    def fresh_cache():
        kv = torch.zeros(NB, 2, BS, KVH, 68, dtype=torch.uint8, device=dev)
        kn = torch.zeros(L, NB, BS, KVH, device=dev)
        vn = torch.zeros_like(kn)
        for s in range(S):
            n = int(hist[s])
            slots = t(np.array([tables[s, p // BS] * BS + p % BS for p in range(n)]), dev)
            g = torch.Generator(device=dev).manual_seed(100 + s)
            akv.fused_tq4_kv_update(torch.randn(n, KVH, 128, device=dev, generator=g).half(), slots, kv[:, 0], kn[0],
                                    tq.rotation, tq.boundaries_inner)
            akv.fused_tq4_kv_update(torch.randn(n, KVH, 128, device=dev, generator=g).half(), slots, kv[:, 1], vn[0],
                                    tq.rotation, tq.boundaries_inner)
        return kv, kn, vn

    new_slots = t(np.array([tables[s, hist[s] // BS] * BS + hist[s] % BS for s in range(S)], dtype=np.int64), dev)
    bt, sl = t(tables, dev), t((hist + 1).astype(np.int32), dev)
    scale = 1 / math.sqrt(128)

    def inputs(seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        return tuple(torch.randn(S, n, 128, device=dev, generator=g).half() for n in (QH, KVH, KVH))

    def run(q, k, v, kv, kn, vn, out):
        return torch.ops.tq.decode_step(q, k, v, kv, out, kn, vn, new_slots, bt, sl, 0, QH, KVH, 128, scale, S)

    # eager results for three different steps, each on a cache of its own
    want = []
    for seed in (1, 2, 3):
        kv, kn, vn = fresh_cache()
        out = torch.zeros(S, QH, 128, dtype=torch.float16, device=dev)
        run(*inputs(seed), kv, kn, vn, out)
        want.append((out.clone(), kv.clone(), kn.clone()))
    # one graph over static tensors
    kv, kn, vn = fresh_cache()
    sq, sk, sv = (x.clone() for x in inputs(1))
    sout = torch.zeros(S, QH, 128, dtype=torch.float16, device=dev)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run(sq, sk, sv, kv, kn, vn, sout)          # warm-up outside the capture (workspaces, tables)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(sq, sk, sv, kv, kn, vn, sout)
    for rep in range(2):
        for i, seed in enumerate((1, 2, 3)):
            q, k, v = inputs(seed)
            sq.copy_(q); sk.copy_(k); sv.copy_(v)
            sout.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(sout, want[i][0]), (rep, seed)
            assert torch.equal(kv, want[i][1]) and torch.equal(kn, want[i][2])
            _ = (torch.randn(1 << 16, device=dev) * 2).sum().item()       # unrelated eager work between replays


@pytest.mark.parametrize("bits", [4, 3])
def test_one_object_across_batch_sizes(golden, dev, bits):
    """One TQPagedAttention (one workspace) serves calls at batch sizes 6, 2, 6, 4, 8, 4, as a server
    that records one graph per batch size does: the cached lookup tables sit at a place in the
    workspace that no batch size moves, so a call at another batch size cannot overwrite them
    behind their validity tag.  Every call is checked against the oracle."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(900 + bits)
    NB, KVH, QH = 64, 8, 32
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, KVH, bits)
    attn = akv.TQPagedAttention(tq, num_query_heads=QH)
    for S in (6, 2, 6, 4, 8, 4):
        ctx = rng.integers(1, 200, size=S).astype(np.int64)
        width = 16
        tables = np.stack([rng.permutation(NB)[:width] for _ in range(S)]).astype(np.int64)
        q = rng.standard_normal((S, QH, 128)).astype(np.float16)
        out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), block_size=16, num_kv_heads=KVH)
        ref = oracle_out(q, kp, kn, vp, vn, tables, ctx, golden, bits)
        assert within_tol(out.cpu().numpy(), ref), f"batch size {S}"
        assert attn.last_call_status() == 0


def test_corrupt_table_entry_stays_inside_the_cache(golden, dev):
    """Table entries inside a context are clamped into [0, num_blocks): a negative or huge entry
    reads a wrong block of the cache, never memory outside it.  The result equals the oracle's on
    the clamped table."""
    tq = make_tq(golden, dev, 4)
    rng = np.random.default_rng(77)
    NB, KVH, QH = 32, 8, 32
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, KVH, 4)
    ctx = np.array([100, 64], dtype=np.int64)
    tables = np.stack([rng.permutation(NB)[:8] for _ in range(2)]).astype(np.int64)
    tables[0, 2] = -5
    tables[1, 1] = 10 ** 9
    q = rng.standard_normal((2, QH, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, num_query_heads=QH)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), block_size=16, num_kv_heads=KVH)
    ref = oracle_out(q, kp, kn, vp, vn, np.clip(tables, 0, NB - 1), ctx, golden, 4)
    assert within_tol(out.cpu().numpy(), ref)


def _poisoned_tail(rng, kp, kn, vp, vn, tables, ctx, block_size):
    """Rows past each context in its last block, and every block no table names: codes 0xFF, norms NaN / +-Inf."""
    NB = kp.shape[0]
    used = np.zeros(NB, dtype=bool)
    bad = np.array([np.nan, np.inf, -np.inf, -1.0], dtype=np.float32)
    for s_, c_ in enumerate(ctx):
        nb = -(-int(c_) // block_size)
        used[tables[s_, :nb]] = True
    for s_, c_ in enumerate(ctx):
        nb = -(-int(c_) // block_size)
        r = int(c_) % block_size
        if nb and r:
            b = int(tables[s_, nb - 1])
            for x in (kp, vp):
                x[b, r:] = 0xFF
            for x in (kn, vn):
                x[b, r:] = torch.from_numpy(rng.choice(bad, size=tuple(x[b, r:].shape))).to(x.device)
    free = torch.from_numpy(np.nonzero(~used)[0]).to(kp.device)
    for x in (kp, vp):
        x[free] = 0xFF
    for x in (kn, vn):
        x[free] = float("nan")


@pytest.mark.parametrize("bits,block_size", [(4, 16), (3, 16), (2, 16), (4, 32), (4, 8), (3, 8)])
def test_rows_past_the_context_may_hold_anything(golden, dev, bits, block_size):
    """The reference reads positions below context_len only (fused_attention.py:166): whatever lies in the
    rest of a sequence's last block, or in blocks that no table names (norms from torch.empty, stale codes),
    must not reach the result.  Blocks of 16 / 32 run the matrix-core kernel, blocks of 8 the general one."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(4100 + bits + block_size)
    NB, KVH, QH = 120, 8, 32
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, KVH, bits, block_size=block_size)
    ctx = np.array([1, block_size - 1, block_size + 1, 3 * block_size, 33 * block_size + 5, 17, 0], dtype=np.int64)
    width = 40
    tables = np.zeros((len(ctx), width), dtype=np.int64)
    perm = rng.permutation(NB)
    off = 0
    for s_, c_ in enumerate(ctx):
        nb = -(-int(c_) // block_size)
        tables[s_, :nb] = perm[off:off + nb]
        off += nb
    q = rng.standard_normal((len(ctx), QH, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, QH)
    clean = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), block_size=block_size)
    ref = oracle_out(q, kp, kn, vp, vn, tables, ctx, golden, bits, block_size=block_size)
    _poisoned_tail(rng, kp, kn, vp, vn, tables, ctx, block_size)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev), block_size=block_size)
    assert bool(torch.isfinite(out).all())
    assert torch.equal(out, clean)
    assert within_tol(out.cpu().numpy(), ref)


@pytest.mark.parametrize("bits", [4, 3, 2])
@pytest.mark.parametrize("case", ["huge", "tiny", "mixed"])
def test_value_norms_far_outside_the_float16_range(golden, dev, bits, case):
    """float32 / bfloat16 inputs reach value norms that no float16 can hold (128 coordinates of 65504 already have
    norm 7.4e5).  The weights of the value product are carried relative to the running maximum of
    score + log2 |v|, so the result keeps its relative accuracy whatever the size of the norms: value vectors
    scaled to norms of 1e5..1e7, of 1e-7..1e-5, and a mix of both in one sequence, float32 queries and outputs
    against the float64 oracle, relative to the largest output of the (sequence, head)."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(7300 + bits)
    NB, KVH, QH = 80, 8, 32
    T = NB * 16
    keys = kv_like(rng, (T, KVH, 128)).astype(np.float32)
    vals = rng.standard_normal((T, KVH, 128)).astype(np.float32)
    vals /= np.linalg.norm(vals, axis=-1, keepdims=True)
    lo, hi = {"huge": (5, 7), "tiny": (-7, -5), "mixed": (-7, 7)}[case]
    vals *= (10.0 ** rng.uniform(lo, hi, size=(T, KVH, 1))).astype(np.float32)
    P = tq._packed_dim
    kp = torch.zeros(NB, 16, KVH, P, dtype=torch.uint8, device=dev)
    vp = torch.zeros_like(kp)
    kn = torch.zeros(NB, 16, KVH, device=dev)
    vn = torch.zeros_like(kn)
    slots = torch.arange(T, device=dev)
    akv.fused_kv_update(t(keys, dev), slots, kp, kn, tq.rotation, tq.boundaries_inner, bits, 16)
    vdev = t(vals, dev) if case != "huge" else t(vals, dev).bfloat16()
    akv.fused_kv_update(vdev, slots, vp, vn, tq.rotation, tq.boundaries_inner, bits, 16)
    assert float(vn.max()) > (1e5 if case != "tiny" else 0) and float(vn.max()) < (1e-4 if case == "tiny" else 1e8)
    ctx = np.array([1000, 37, 1280, 1], dtype=np.int64)
    tables = np.stack([rng.permutation(NB) for _ in ctx]).astype(np.int64)
    q = rng.standard_normal((len(ctx), QH, 128)).astype(np.float32)
    attn = akv.TQPagedAttention(tq, QH)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev)).cpu().numpy().astype(np.float64)
    ref = oracle_out(q, kp, kn, vp, vn, tables, ctx, golden, bits)
    assert np.all(np.isfinite(out))
    scale = np.abs(ref).max(axis=-1, keepdims=True)
    rel = np.max(np.abs(out - ref) / scale)
    print(f"[attn value norms {case}] bits={bits} max|out|={np.abs(ref).max():.3e} max relative diff={rel:.2e}")
    assert rel <= 5e-4
    assert attn.last_call_status() == 0


@pytest.mark.parametrize("bits", [4, 2])
@pytest.mark.parametrize("S,empty_every", [(40, 0), (33, 2), (64, 0), (64, 3), (65, 0), (20, 0), (32, 0), (1, 0)])
def test_partition_of_the_block_axis_by_batch_shape(golden, dev, bits, S, empty_every):
    """The three ways the prologue cuts the block axis among the workgroups -- whole workgroups per sequence (few
    non-empty sequences), equal ranges with the sequences held by one wavefront (up to 64 sequences), equal
    ranges through the general scan (more) -- with empty sequences in between, sequences of one token and
    lengths that leave the last workgroup of a sequence a single block: every sequence against the oracle."""
    tq = make_tq(golden, dev, bits)
    rng = np.random.default_rng(8800 + 7 * S + bits + empty_every)
    NB, KVH, QH = 400, 8, 32
    kp, kn, vp, vn = build_cache(rng, tq, dev, NB, KVH, bits)
    ctx = rng.integers(1, 2500, size=S).astype(np.int64)
    ctx[rng.integers(0, S)] = 1
    ctx[rng.integers(0, S)] = 16 * 33 + 1
    if empty_every:
        ctx[::empty_every] = 0
    width = int(-(-ctx.max() // 16))
    tables = np.full((S, width), -9, dtype=np.int32)
    for s_, c_ in enumerate(ctx):
        nb = -(-int(c_) // 16)
        tables[s_, :nb] = rng.integers(0, NB, size=nb)        # blocks may repeat between sequences: only reads
    q = rng.standard_normal((S, QH, 128)).astype(np.float16)
    attn = akv.TQPagedAttention(tq, QH)
    out = attn.forward(t(q, dev), kp, kn, vp, vn, t(tables, dev), t(ctx, dev)).cpu().numpy()
    refs = oracle_rows_of_batch(q, kp, kn, vp, vn, np.maximum(tables, 0), ctx, golden, bits, range(S))
    for s_, r_ in refs.items():
        assert within_tol(out[s_], r_), f"sequence {s_} of {S} (ctx {ctx[s_]})"
    assert attn.last_call_status() == 0

"""Randomly drawn VALID shapes of every entry point of the hot path against the oracle: the hand-picked cases of
the other test files fix the shapes someone thought of; these draw bit width, block size, head counts, GQA
ratio, batch size, context lengths (empty, shorter than a block, filling the table, all equal), table and length
dtypes, query dtype, row pitch, coefficient width ... from a seeded generator, a few dozen draws per path.
Every case prints its parameters before it runs."""
import math

import numpy as np
import pytest
import torch

import aitherkvcache_amd as akv
from aitherkvcache_amd.triattention import TriAttention, TriAttentionConfig
from oracle import tq_oracle as O
from tests.test_gpu_attention import within_tol
from tests.test_gpu_hybrid import build_cache as hybrid_cache, params as hybrid_params
from tests.util import kv_like

pytestmark = pytest.mark.gpu


def t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def as_dtype(x32, which, dev):
    """float32 host array -> device tensor of the drawn dtype, and what it holds read back as float32."""
    d = t(x32, dev).to((torch.float32, torch.float16, torch.bfloat16)[which])
    return d, d.float().cpu().numpy()


def draw_contexts(rng, S, max_tokens, block_size):
    mode = int(rng.integers(0, 4))
    if mode == 0:
        ctx = rng.integers(0, max_tokens + 1, S)
    elif mode == 1:
        ctx = rng.integers(0, min(max_tokens, 3 * block_size) + 1, S)
    elif mode == 2:
        ctx = np.where(rng.random(S) < 0.5, 0, rng.integers(1, max_tokens + 1, S))
    else:
        ctx = np.full(S, int(rng.integers(1, max_tokens + 1)))
    return ctx.astype(np.int64)


@pytest.mark.parametrize("seed", range(4))
def test_paged_attention_random_shapes(golden, dev, seed):
    R = golden["rotation_d128_seed42"]
    for case in range(20):
        rng = np.random.default_rng(7_000_000 + 1000 * seed + case)
        bits = int(rng.choice([2, 3, 4]))
        bs = int(rng.choice([8, 16, 16, 16, 32, 32]))
        kvh = int(rng.choice([1, 2, 3, 4, 5, 8, 8, 12, 16]))
        gqa = int(rng.choice([1, 2, 3, 4, 4, 5, 8, 12, 16, 20]))
        if kvh * gqa > 96:
            gqa = max(1, 96 // kvh)
        qh = kvh * gqa
        S = int(rng.choice([1, 2, 3, 5, 8, 16, 17, 31, 32, 33, 40, 64, 65, 70]))
        NB = int(rng.integers(4, 160))
        pad = int(rng.choice([0, 0, 4]))                 # rows of packed + 4 bytes: the serving layout
        qdt = int(rng.integers(0, 3))
        it = (torch.int32, torch.int64)[int(rng.integers(0, 2))]
        ct = (torch.int32, torch.int64)[int(rng.integers(0, 2))]
        ctx = draw_contexts(rng, S, NB * bs, bs)
        width = max(1, int(-(-ctx.max() // bs)) + int(rng.integers(0, 3)))
        print(f"[random attn {seed}/{case}] bits={bits} bs={bs} kvh={kvh} qh={qh} S={S} NB={NB} pad={pad} qdt={qdt} "
              f"tables={it} lens={ct} tokens={int(ctx.sum())} width={width}", flush=True)
        tq = akv.TurboQuant(head_dim=128, bits=bits, device=str(dev))
        tq.rotation = t(R, dev)
        P = tq._packed_dim
        kp = torch.zeros(NB, bs, kvh, P + pad, dtype=torch.uint8, device=dev)
        vp = torch.zeros_like(kp)
        kn = torch.zeros(NB, bs, kvh, device=dev)
        vn = torch.zeros_like(kn)
        slots = torch.arange(NB * bs, device=dev)
        for x, p_, n_ in ((kv_like(rng, (NB * bs, kvh, 128)), kp, kn), (kv_like(rng, (NB * bs, kvh, 128)), vp, vn)):
            akv.fused_kv_update(t(x, dev), slots, p_[..., :P], n_, tq.rotation, tq.boundaries_inner, bits, bs)
        tables = np.full((S, width), int(rng.choice([-7, 10 ** 6, 0])), dtype=np.int64)    # padding is never read
        for s, c_ in enumerate(ctx):
            nb = -(-int(c_) // bs)
            shared = rng.random() < 0.3 or nb > NB       # blocks may repeat inside and across sequences
            tables[s, :nb] = rng.integers(0, NB, nb) if shared else rng.permutation(NB)[:nb]
        q32 = rng.standard_normal((S, qh, 128)).astype(np.float32) * float(rng.choice([0.3, 1.0, 3.0]))
        qd, qhost = as_dtype(q32, qdt, dev)
        out = akv.TQPagedAttention(tq, num_query_heads=qh).forward(
            qd, kp[..., :P], kn, vp[..., :P], vn, t(tables, dev).to(it), t(ctx, dev).to(ct), block_size=bs, num_kv_heads=kvh)
        assert out.dtype == qd.dtype
        c, _, _ = O.get_codebook(128, bits)
        ref = O.paged_attention(qhost, kp.cpu().numpy()[..., :P], kn.cpu().numpy(), vp.cpu().numpy()[..., :P],
                                vn.cpu().numpy(), tables, ctx, R, c, bits, block_size=bs, dtype=np.float64, cast_output=False)
        got = out.float().cpu().numpy().astype(np.float64)
        err = np.abs(got - ref)
        assert np.all(np.isfinite(got)) and np.all(got[ctx == 0] == 0)
        if qdt == 0:        # float32 in and out: the arithmetic alone
            assert np.all(err <= 1e-3 + 2e-4 * np.abs(ref)), err.max()
        elif qdt == 1:
            assert within_tol(got, ref), err.max()
        else:               # 2e-3 plus half a bfloat16 unit in the last place of the output
            assert np.all(err <= 2e-3 + 2.0 ** -8 * np.abs(ref)), err.max()


@pytest.mark.parametrize("seed", range(2))
def test_hybrid_attention_random_shapes(golden, dev, seed):
    hp = hybrid_params(golden)
    for case in range(15):
        rng = np.random.default_rng(8_000_000 + 1000 * seed + case)
        kvh = int(rng.choice([1, 2, 3, 4, 8, 8]))
        gqa = int(rng.choice([1, 2, 3, 4, 4, 4, 8, 12, 20]))
        if kvh * gqa > 64:
            gqa = max(1, 64 // kvh)
        qh = kvh * gqa
        bs = int(rng.choice([8, 16, 16, 32]))
        S = int(rng.choice([1, 2, 5, 16, 33, 40, 64, 65]))
        NB = int(rng.integers(3, 120))
        ctx = draw_contexts(rng, S, NB * bs, bs)
        qdt = int(rng.integers(0, 3))
        print(f"[random tq35 {seed}/{case}] kvh={kvh} qh={qh} bs={bs} S={S} NB={NB} qdt={qdt} tokens={int(ctx.sum())}", flush=True)
        h = akv.HybridTurboQuant(device=str(dev))
        h.calibrate_uniform(num_kv_heads=kvh)
        kc, vc, _, _ = hybrid_cache(rng, h, dev, NB, kvh, BS=bs)
        width = max(1, int(-(-ctx.max() // bs)) + 1)
        tables = np.full((S, width), -3, dtype=np.int64)
        for s, c_ in enumerate(ctx):
            nb = -(-int(c_) // bs)
            tables[s, :nb] = rng.integers(0, NB, nb)
        qd, qhost = as_dtype(rng.standard_normal((S, qh, 128)).astype(np.float32), qdt, dev)
        scale = 1 / math.sqrt(128)
        it = torch.int32 if rng.random() < 0.5 else torch.int64
        out = akv.HybridPagedAttention(h, qh).forward(qd, kc, vc, t(tables, dev).to(it), t(ctx, dev), block_size=bs, scale=scale)
        ref = O.hybrid_paged_attention(qhost, kc.cpu().numpy(), vc.cpu().numpy(), np.where(tables >= 0, tables, 0), ctx, hp,
                                       scale, block_size=bs, dtype=np.float64)
        got = out.float().cpu().numpy().astype(np.float64)
        out_ulp = (0.0, 2.0 ** -11, 2.0 ** -8)[qdt]
        assert np.all(np.isfinite(got)) and np.all(got[ctx == 0] == 0)
        assert np.all(np.abs(got - ref) <= 3e-4 + out_ulp * np.abs(ref)), np.abs(got - ref).max()


@pytest.mark.parametrize("seed", range(2))
def test_triattention_random_shapes(dev, seed):
    for case in range(25):
        rng = np.random.default_rng(9_000_000 + 1000 * seed + case)
        D = int(rng.choice([32, 64, 128, 128, 128]))
        F = min(int(rng.choice([4, 7, 12, 12, 12, 16, 20])), D // 2)
        KVH = int(rng.choice([1, 2, 4, 8, 8, 16]))
        QH = KVH * int(rng.choice([1, 2, 3, 4, 4, 8]))
        B = int(rng.integers(1, 5))
        S = int(rng.choice([1, 2, 63, 64, 65, 130, 333, 1000, 2500]))
        bits = int(rng.choice([4, 4, 4, 8, 16]))
        pre = bool(rng.random() < 0.8)
        base = float(rng.choice([1e4, 1e6]))
        qdt = int(rng.integers(0, 3))
        print(f"[random tri {seed}/{case}] D={D} F={F} KVH={KVH} QH={QH} B={B} S={S} bits={bits} pre_rope={pre} base={base} "
              f"qdt={qdt}", flush=True)
        cfg = TriAttentionConfig(head_dim=D, num_freqs=F, coeff_bits=bits, num_kv_heads=KVH, num_query_heads=QH,
                                 rope_base=base, pre_rope=pre)
        tri = TriAttention(cfg, device=str(dev))
        pair_std = (np.arange(D // 2) + 1.0) ** -0.75
        keys = (rng.standard_normal((B, S, KVH, D // 2, 2)) * pair_std[:, None]).reshape(B, S, KVH, D).astype(np.float16)
        vals = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
        k_enc, v_enc = tri.encode_kv(t(keys, dev), t(vals, dev))
        k_ref, v_ref = O.spectral_encode(keys, F, bits), O.spectral_encode(vals, F, bits)
        for enc, ref in ((k_enc, k_ref), (v_enc, v_ref)):      # the write side, byte for byte
            assert np.array_equal(enc.indices.cpu().numpy(), ref[0])
            assert np.array_equal(enc.packed.cpu().numpy().view(np.uint8), ref[1].view(np.uint8))
            assert np.array_equal(enc.scales.cpu().numpy(), ref[2])
        qd, qhost = as_dtype(rng.standard_normal((B, QH, D)).astype(np.float32), qdt, dev)
        theta = tri._theta.cpu().numpy()
        if rng.random() < 0.5:
            qpos = rng.integers(S, 40000, size=B)
            kpos = np.sort(rng.integers(0, 32768, size=(B, S)), axis=-1)
            out = tri.decode_step(qd, k_enc, v_enc, t(qpos, dev), t(kpos, dev)).cpu().numpy()
            ref = O.tri_decode_step(qhost, k_ref, v_ref, theta, qpos, kpos, coeff_bits=bits, pre_rope=pre)
        else:
            out = tri.decode_step(qd, k_enc, v_enc).cpu().numpy()
            ref = O.tri_decode_step(qhost, k_ref, v_ref, theta, coeff_bits=bits, pre_rope=pre)
        assert np.all(np.isfinite(out)) and np.max(np.abs(out - ref)) <= 2e-5


@pytest.mark.parametrize("seed", range(2))
def test_codec_random_shapes(dev, seed):
    """Flat encode / decode over leading shapes of zero to two axes (an empty batch and a single vector among
    them), the three input dtypes, rows with a pitch of their own and every head dimension the kernels take.
    The wide heads (256, 512: float32 sums of that many terms in the kernel and in the oracle alike) are given
    32 float32 units in the last place around a decision boundary instead of 16."""
    for case in range(40):
        rng = np.random.default_rng(10_000_000 + 1000 * seed + case)
        bits = int(rng.choice([2, 3, 4]))
        d = int(rng.choice([64, 128, 128, 256, 512]))
        lead = [(), (int(rng.integers(0, 7)),), (int(rng.integers(1, 5)), int(rng.integers(1, 9))),
                (int(rng.integers(1, 3000)),)][int(rng.integers(0, 4))]
        which = int(rng.integers(0, 3))
        strided = bool(rng.random() < 0.3) and bool(lead)
        print(f"[random codec {seed}/{case}] bits={bits} d={d} lead={lead} dtype={which} strided={strided}", flush=True)
        tq = akv.TurboQuant(head_dim=d, bits=bits, device=str(dev))
        Rm = tq.rotation.cpu().numpy()
        n = int(np.prod(lead)) if lead else 1
        x = (rng.standard_normal(lead + (d,)) * rng.lognormal(0, 0.7, lead + (1,))).astype(np.float32)
        if n > 2:
            x.reshape(-1, d)[1] = 0.0
        xd, xh = as_dtype(x, which, dev)
        if strided:
            buf = torch.zeros(lead + (d + 8,), dtype=xd.dtype, device=dev)
            buf[..., :d] = xd
            xd = buf[..., :d]
        packed, norms = tq.encode(xd)
        assert packed.shape == lead + (d * bits // 8,) and norms.shape == lead
        dec = tq.decode(packed, norms)
        assert dec.shape == xd.shape
        if n == 0:
            continue
        rep = O.encode_parity_report(packed.cpu().numpy().reshape(-1, packed.shape[-1]), norms.cpu().numpy().reshape(-1),
                                     xh.reshape(-1, d), Rm, bits)
        assert rep["mismatching"] <= max(3, int(2e-5 * n * d)) and rep["max_code_step"] <= 1, rep
        assert rep["max_ulps_from_boundary"] <= (16 if d <= 128 else 32), rep
        assert rep["norm_max_rel_diff"] <= 1e-6, rep
        cen, _, _ = O.get_codebook(d, bits)
        ref = O.decode(packed.cpu().numpy(), norms.cpu().numpy(), Rm, cen, bits).astype(np.float32)
        assert np.max(np.abs(dec.float().cpu().numpy() - ref)) <= 2e-3 * max(1.0, float(np.abs(ref).max()))


@pytest.mark.parametrize("seed", range(2))
def test_paged_update_random_shapes(golden, dev, seed):
    """Distinct slots, some negative and some past the cache (both skipped), a block limit below the cache size,
    rows with a pitch of their own: written rows against the oracle, every other byte and norm untouched."""
    R = golden["rotation_d128_seed42"]
    for case in range(40):
        rng = np.random.default_rng(11_000_000 + 1000 * seed + case)
        bits = int(rng.choice([2, 3, 4]))
        bs = int(rng.choice([8, 16, 32]))
        kvh = int(rng.choice([1, 2, 8]))
        NB = int(rng.integers(2, 60))
        T = int(rng.integers(0, min(400, NB * bs + 20)))
        pad = int(rng.choice([0, 4]))
        which = int(rng.integers(0, 3))
        max_blocks = int(rng.choice([0, NB, max(1, NB // 2)]))
        print(f"[random update {seed}/{case}] bits={bits} bs={bs} kvh={kvh} NB={NB} T={T} pad={pad} dtype={which} "
              f"max_blocks={max_blocks}", flush=True)
        tq = akv.TurboQuant(head_dim=128, bits=bits, device=str(dev))
        tq.rotation = t(R, dev)
        P = tq._packed_dim
        xd, xh = as_dtype(kv_like(rng, (T, kvh, 128)).astype(np.float32), which, dev)
        slots = rng.permutation(NB * bs + 20)[:T].astype(np.int64) - 10
        kp = torch.full((NB, bs, kvh, P + pad), 0xAB, dtype=torch.uint8, device=dev)
        kn = torch.full((NB, bs, kvh), -5.0, device=dev)
        akv.fused_kv_update(xd, t(slots, dev), kp[..., :P], kn, tq.rotation, tq.boundaries_inner, bits, bs, max_blocks)
        ref_p = np.full((NB, bs, kvh, P), 0xAB, np.uint8)
        ref_n = np.full((NB, bs, kvh), -5.0, np.float32)
        _, b_in, _ = O.get_codebook(128, bits)
        O.kv_update(xh, slots, ref_p, ref_n, R, b_in, bs, max_blocks, bits)
        gp, gn = kp.cpu().numpy(), kn.cpu().numpy()
        untouched = ref_n == -5.0
        assert np.array_equal(gn == -5.0, untouched)
        assert np.all(gp[..., P:] == 0xAB) and np.all(gp[untouched][..., :P] == 0xAB)
        ca = O._UNPACK[bits](gp[..., :P].reshape(-1, P), 128)
        cb = O._UNPACK[bits](ref_p.reshape(-1, P), 128)
        assert int(np.sum(ca != cb)) <= max(3, int(2e-5 * ca.size))
        assert int(np.max(np.abs(ca.astype(int) - cb.astype(int)), initial=0)) <= 1
        if T:
            assert np.max(np.abs(gn - ref_n) / np.maximum(np.abs(ref_n), 1e-30)) <= 1e-6

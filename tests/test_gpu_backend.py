"""TurboQuantBackend / TurboQuantImpl driven the way vLLM drives an attention backend (do_kv_cache_update,
then forward with an attention-metadata object), without vLLM: a namespace stands for the metadata, and the
dense paged attention of the prefill path (vLLM's kernel) is replaced by a recorder.  What the impl writes
into the cache and returns from decode is checked against the oracle."""
import math
import types

import numpy as np
import pytest
import torch

from aitherkvcache_amd.vllm import backend as B
from oracle import tq_oracle as O
from tests.util import check_codes, kv_like

pytestmark = pytest.mark.gpu

BS, KVH, QH, NB, LAYERS = 16, 2, 8, 24, 2
TOL = 2e-3


def t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def within_tol(got, ref64):
    got = np.asarray(got, dtype=np.float64)
    return bool(np.all(np.abs(got - ref64) <= TOL + 2.0 ** -11 * np.abs(ref64)))


def meta(dev, slots, tables, seq_lens, num_actual, max_query_len, query_lens=None):
    query_lens = query_lens if query_lens is not None else [1] * len(seq_lens)
    return types.SimpleNamespace(
        slot_mapping=t(np.asarray(slots, dtype=np.int64), dev), block_table=t(np.asarray(tables, dtype=np.int32), dev),
        seq_lens=t(np.asarray(seq_lens, dtype=np.int32), dev), num_actual_tokens=num_actual,
        max_query_len=max_query_len, max_seq_len=int(max(seq_lens)),
        query_start_loc=t(np.concatenate([[0], np.cumsum(query_lens)]).astype(np.int32), dev))


@pytest.fixture
def impl_cls():
    cls = B.TurboQuantBackend.get_impl_cls()
    cls.reset_class_state()
    yield cls
    cls.reset_class_state()
    cls._dense_paged_attention = staticmethod(B._vllm_unified_attention)
    cls._INIT_AFTER_FORWARDS = 2


def make_layers(cls, golden, dev, dtype_name):
    layers = [cls(QH, 128, 1 / math.sqrt(128), num_kv_heads=KVH, kv_cache_dtype=dtype_name) for _ in range(LAYERS)]
    tq = layers[0]._quantizer(dev)
    if hasattr(tq, "rotation"):
        tq.rotation = torch.from_numpy(golden["rotation_d128_seed42"]).to(dev)
    return layers, tq


def slots_of(tables, s, start, stop):
    return [int(tables[s][p // BS]) * BS + p % BS for p in range(start, stop)]


def hybrid_params(golden, tq25=None):
    if tq25 is not None:
        books = ((tq25["g0_centroids"], tq25["g0_boundaries"]), (tq25["g1_centroids"], tq25["g1_boundaries"]))
        return O.HybridParams(tq25["g0_had"], tq25["g1_had"], tq25["g0_qjl"], tq25["g1_qjl"], codebooks=books, mode="tq25")
    books = tuple((golden[f"hyb_centroids_64_{k}"], golden[f"hyb_boundaries_64_{k}"]) for k in (3, 2))
    return O.HybridParams(golden["hyb_g0_had_signs"], golden["hyb_g1_had_signs"],
                          golden["hyb_g0_qjl_signs"], golden["hyb_g1_qjl_signs"], codebooks=books)


def test_backend_class_surface():
    bk = B.TurboQuantBackend
    assert bk.get_name() == "CUSTOM" and bk.accept_output_buffer and not bk.forward_includes_kv_cache_update
    assert bk.get_kv_cache_shape(7, 16, 8, 128) == (7, 2, 16, 8, 128)
    assert bk.get_kv_cache_shape(7, 16, 8, 128, "tq-t4nc") == (7, 2, 16, 8, 68)
    assert bk.get_supported_head_sizes() == [64, 96, 128, 256, 512]
    assert bk.get_impl_cls() is B.TurboQuantImpl
    with pytest.raises(RuntimeError, match="vLLM"):
        bk.get_builder_cls()


@pytest.mark.parametrize("bits", [4, 3])
def test_primary_uniform_prefill_then_decode(golden, dev, impl_cls, bits):
    """Two sequences: a prefill chunk each (37 and 20 tokens, plus one padding row), then a decode step,
    all on layer 1 of 2.  Cache rows and norms against O.kv_update, the prefill block buffers against
    O.decode, the decode output against the oracle's attention over the written cache."""
    layers, tq = make_layers(impl_cls, golden, dev, f"tq-t{bits}nc")
    impl = layers[1]
    R = golden["rotation_d128_seed42"]
    cen, bnd, _ = O.get_codebook(128, bits)
    P = tq._packed_dim
    rng = np.random.default_rng(900 + bits)
    kv_cache = torch.zeros(*B.TurboQuantBackend.get_kv_cache_shape(NB, BS, KVH, 128, f"tq-t{bits}nc"),
                           dtype=torch.uint8, device=dev)
    tables = np.array([[5, 11, 2, 0], [20, 7, 0, 0]], dtype=np.int32)
    lens = [37, 20]
    keys = [kv_like(rng, (n + 1, KVH, 128)) for n in lens]
    vals = [kv_like(rng, (n + 1, KVH, 128)) for n in lens]

    # ---- prefill chunk: 57 real rows and one padding row (slot -1)
    slots = slots_of(tables, 0, 0, 37) + slots_of(tables, 1, 0, 20) + [-1]
    k = np.concatenate([keys[0][:37], keys[1][:20], np.ones((1, KVH, 128), np.float16)])
    v = np.concatenate([vals[0][:37], vals[1][:20], np.ones((1, KVH, 128), np.float16)])
    q = rng.standard_normal((58, QH, 128)).astype(np.float16)
    md = meta(dev, slots, tables, lens, 57, 37, query_lens=lens)
    seen = {}

    def recorder(impl_, q_, k_buf, v_buf, out, md_):
        seen.update(q=q_.clone(), k=k_buf.clone(), v=v_buf.clone(), md=md_)
        out.fill_(0.25)
    impl_cls._dense_paged_attention = staticmethod(recorder)
    impl.do_kv_cache_update(None, t(k, dev), t(v, dev), kv_cache, md.slot_mapping)
    out = torch.full((58, QH * 128), 7.0, dtype=torch.float16, device=dev)
    assert impl.forward(None, t(q, dev).view(58, QH * 128), t(k, dev), t(v, dev), kv_cache, md, output=out) is out
    assert torch.all(out[:57] == 0.25) and torch.all(out[57] == 7.0)         # padding row untouched
    assert seen["q"].shape == (57, QH, 128) and seen["k"].dtype == torch.bfloat16 and seen["md"] is md

    ref_p = np.zeros((NB, BS, KVH, P), np.uint8)
    ref_n = np.zeros((NB, BS, KVH), np.float32)
    for li, (x, which) in enumerate(((k, 0), (v, 1))):
        ref_p[:] = 0
        ref_n[:] = 0
        O.kv_update(x, np.asarray(slots), ref_p, ref_n, R, bnd, block_size=BS, bits=bits)
        norms = (impl_cls._primary_k_norms, impl_cls._primary_v_norms)[which]
        assert norms.shape == (LAYERS, NB, BS, KVH) and torch.all(norms[0] == 0)
        got_p = kv_cache[:, which, :, :, :P].cpu().numpy()
        got_n = norms[1].cpu().numpy()
        order = np.argsort(np.asarray(slots[:57]))                          # rows in slot order, like the cache
        written = ref_n > 0
        assert np.array_equal(got_n > 0, written)
        check_codes(got_p[written], got_n[written], x[:57][order].reshape(-1, 128), R, bits, ref_p[written], ref_n[written])
        assert np.all(got_p[~written] == 0) and torch.all(kv_cache[..., P:] == 0)
        # block buffers of the prefill path: decoded history, except the chunk's own rows (uncompressed)
        buf = (seen["k"], seen["v"])[which].float().cpu().numpy()
        for s in range(2):
            for p in range(lens[s]):
                b, o = int(tables[s][p // BS]), p % BS
                row = (keys, vals)[which][s][p]
                assert np.array_equal(buf[b, o], torch.from_numpy(row).bfloat16().float().numpy())
        # a row of an addressed block that the chunk did not write holds the decoded (zero) cache row
        assert np.all(buf[int(tables[1][1]), 5:] == 0)

    # ---- history rows come back decoded on a later chunk: second chunk for sequence 1 (tokens 20..20)
    md2 = meta(dev, slots_of(tables, 1, 20, 21), tables[1:2], [21], 1, 2, query_lens=[1])
    k2, v2 = keys[1][20:21], vals[1][20:21]
    impl.do_kv_cache_update(None, t(k2, dev), t(v2, dev), kv_cache, md2.slot_mapping)
    out2 = torch.zeros(1, QH * 128, dtype=torch.float16, device=dev)
    impl.forward(None, t(q[:1], dev).view(1, -1), t(k2, dev), t(v2, dev), kv_cache, md2, output=out2)
    kn = impl_cls._primary_k_norms[1].cpu().numpy()
    b0 = int(tables[1][0])
    dec = O.decode(kv_cache[b0, 0, :, :, :P].cpu().numpy(), kn[b0], R, cen, bits).astype(np.float32)
    got = seen["k"][b0].float().cpu().numpy()
    assert np.all(np.abs(got - dec) <= 2e-3 + np.abs(dec) * 2.0 ** -8)        # bf16 rounding of the buffer

    # ---- decode step: token 37 of sequence 0, token 21 of sequence 1
    new_slots = slots_of(tables, 0, 37, 38) + slots_of(tables, 1, 21, 22) + [-1]
    kd = np.concatenate([keys[0][37:38], kv_like(rng, (1, KVH, 128)), np.zeros((1, KVH, 128), np.float16)])
    vd = np.concatenate([vals[0][37:38], kv_like(rng, (1, KVH, 128)), np.zeros((1, KVH, 128), np.float16)])
    qd = rng.standard_normal((3, QH, 128)).astype(np.float16)
    mdd = meta(dev, new_slots, tables, [38, 22], 2, 1)
    impl.do_kv_cache_update(None, t(kd, dev), t(vd, dev), kv_cache, mdd.slot_mapping)
    outd = torch.full((3, QH * 128), 3.0, dtype=torch.float16, device=dev)
    impl.forward(None, t(qd, dev).view(3, -1), t(kd, dev), t(vd, dev), kv_cache, mdd, output=outd)
    ref = O.paged_attention(qd[:2], kv_cache[:, 0, :, :, :P].cpu().numpy(), impl_cls._primary_k_norms[1].cpu().numpy(),
                            kv_cache[:, 1, :, :, :P].cpu().numpy(), impl_cls._primary_v_norms[1].cpu().numpy(),
                            tables, np.array([38, 22]), R, cen, bits, block_size=BS, dtype=np.float64, cast_output=False)
    assert within_tol(outd[:2].view(2, QH, 128).cpu().numpy(), ref)
    assert torch.all(outd[2] == 3.0)
    assert float(impl_cls._primary_k_norms[1, tables[0][2], 37 % BS, 0]) > 0        # the step's row was written


def test_primary_decode_without_separate_cache_update(golden, dev, impl_cls):
    """A vLLM release that never calls do_kv_cache_update: forward writes the step's rows and attends in
    one op (tq::decode_step)."""
    layers, tq = make_layers(impl_cls, golden, dev, "tq-t4nc")
    impl = layers[0]
    R = golden["rotation_d128_seed42"]
    cen, bnd, _ = O.get_codebook(128, 4)
    rng = np.random.default_rng(77)
    kv_cache = torch.zeros(NB, 2, BS, KVH, 68, dtype=torch.uint8, device=dev)
    tables = np.array([[9, 1], [3, 0]], dtype=np.int32)
    qs = rng.standard_normal((4, 2, QH, 128)).astype(np.float16)
    for step in range(4):                                   # four decode steps from empty sequences
        slots = slots_of(tables, 0, step, step + 1) + slots_of(tables, 1, step, step + 1)
        md = meta(dev, slots, tables, [step + 1, step + 1], 2, 1)
        k, v = kv_like(rng, (2, KVH, 128)), kv_like(rng, (2, KVH, 128))
        out = torch.zeros(2, QH * 128, dtype=torch.float16, device=dev)
        impl.forward(None, t(qs[step], dev).view(2, -1), t(k, dev), t(v, dev), kv_cache, md, output=out)
        ref = O.paged_attention(qs[step], kv_cache[:, 0, :, :, :64].cpu().numpy(), impl_cls._primary_k_norms[0].cpu().numpy(),
                                kv_cache[:, 1, :, :, :64].cpu().numpy(), impl_cls._primary_v_norms[0].cpu().numpy(),
                                tables, np.array([step + 1, step + 1]), R, cen, 4, block_size=BS, dtype=np.float64,
                                cast_output=False)
        assert within_tol(out.view(2, QH, 128).cpu().numpy(), ref), step
        ref_p = np.zeros((NB, BS, KVH, 64), np.uint8)
        ref_n = np.zeros((NB, BS, KVH), np.float32)
        O.kv_update(k, np.asarray(slots), ref_p, ref_n, R, bnd, block_size=BS, bits=4)
        w = ref_n > 0
        check_codes(kv_cache[:, 0, :, :, :64].cpu().numpy()[w], impl_cls._primary_k_norms[0].cpu().numpy()[w],
                    k[np.argsort(slots)].reshape(-1, 128), R, 4, ref_p[w], ref_n[w])
    assert int((impl_cls._primary_k_norms[0] > 0).sum()) == 4 * 2 * KVH


@pytest.mark.parametrize("mode,row", [("tq35", 64), ("tq25", 44)])
def test_primary_hybrid_decode(golden, tq25, dev, impl_cls, mode, row):
    layers, htq = make_layers(impl_cls, golden, dev, mode)
    impl = layers[1]
    hp = hybrid_params(golden, tq25 if mode == "tq25" else None)
    rng = np.random.default_rng(78)
    kv_cache = torch.zeros(*B.TurboQuantBackend.get_kv_cache_shape(NB, BS, KVH, 128, mode), dtype=torch.uint8, device=dev)
    assert kv_cache.shape[-1] == row
    tables = np.array([[4, 8, 0], [1, 6, 0]], dtype=np.int32)
    hist = 21
    seen = {}
    impl_cls._dense_paged_attention = staticmethod(lambda i, q, kb, vb, out, md: (seen.update(k=kb.clone()), out.zero_()))
    slots = slots_of(tables, 0, 0, hist) + slots_of(tables, 1, 0, hist)
    k, v = kv_like(rng, (2 * hist, KVH, 128)), kv_like(rng, (2 * hist, KVH, 128))
    md = meta(dev, slots, tables, [hist, hist], 2 * hist, hist, query_lens=[hist, hist])
    impl.do_kv_cache_update(None, t(k, dev), t(v, dev), kv_cache, md.slot_mapping)
    out = torch.zeros(2 * hist, QH * 128, dtype=torch.float16, device=dev)
    impl.forward(None, torch.zeros(2 * hist, QH * 128, dtype=torch.float16, device=dev), None, None, kv_cache, md, output=out)
    # prefill buffer = decoded rows (key=None: nothing scattered over them)
    b = int(tables[0][0])
    dec = O.hybrid_decode(kv_cache[b, 0].cpu().numpy(), hp)
    got = seen["k"][b].float().cpu().numpy()
    assert np.all(np.abs(got - dec) <= 2e-3 + np.abs(dec) * 2.0 ** -8)
    # decode step
    new_slots = slots_of(tables, 0, hist, hist + 1) + slots_of(tables, 1, hist, hist + 1)
    kd, vd = kv_like(rng, (2, KVH, 128)), kv_like(rng, (2, KVH, 128))
    qd = rng.standard_normal((2, QH, 128)).astype(np.float16)
    mdd = meta(dev, new_slots, tables, [hist + 1, hist + 1], 2, 1)
    impl.do_kv_cache_update(None, t(kd, dev), t(vd, dev), kv_cache, mdd.slot_mapping)
    outd = torch.zeros(2, QH * 128, dtype=torch.float16, device=dev)
    impl.forward(None, t(qd, dev).view(2, -1), t(kd, dev), t(vd, dev), kv_cache, mdd, output=outd)
    ref = O.hybrid_paged_attention(qd, kv_cache[:, 0].cpu().numpy(), kv_cache[:, 1].cpu().numpy(), tables,
                                   np.array([hist + 1, hist + 1]), hp, impl.scale, dtype=np.float64)
    assert np.max(np.abs(outd.view(2, QH, 128).cpu().numpy().astype(np.float64) - ref)) <= 2e-3
    assert impl_cls._primary_k_norms is None            # hybrid rows carry their norms


def test_shadow_copy_serves_decode(golden, dev, impl_cls, monkeypatch):
    """SHADOW mode: vLLM's cache is not touched; the compressed copy appears once enough forwards have
    run, takes every step's rows, and serves decode when AITHER_TQ_FUSED=1.  Whatever is the parent's job
    raises without vLLM."""
    monkeypatch.setenv("AITHER_TQ_FUSED", "1")
    monkeypatch.delenv("AITHER_TQ_MODE", raising=False)
    monkeypatch.delenv("AITHER_TQ_PRIMARY", raising=False)
    monkeypatch.delenv("AITHER_TQ_BITS", raising=False)
    impl_cls.reset_class_state()
    impl_cls._INIT_AFTER_FORWARDS = 1
    layers = [impl_cls(QH, 128, 1 / math.sqrt(128), num_kv_heads=KVH) for _ in range(LAYERS)]
    assert not impl_cls._tq_primary and impl_cls._fused_enabled and impl_cls._tq_format.bits == 4
    R = golden["rotation_d128_seed42"]
    cen, _, _ = O.get_codebook(128, 4)
    rng = np.random.default_rng(79)
    kv_cache = torch.zeros(NB, 2, BS, KVH, 128, dtype=torch.float16, device=dev)      # vLLM's own cache
    tables = np.array([[2, 3]], dtype=np.int32)
    k, v = kv_like(rng, (20, KVH, 128)), kv_like(rng, (20, KVH, 128))
    md = meta(dev, slots_of(tables, 0, 0, 20), tables, [20], 20, 20, query_lens=[20])
    out = torch.zeros(20, QH * 128, dtype=torch.float16, device=dev)
    for impl in layers:
        impl.do_kv_cache_update(None, t(k, dev), t(v, dev), kv_cache, md.slot_mapping)      # parent's write: no-op here
        with pytest.raises(RuntimeError, match="vLLM"):                                      # prefill is the parent's
            impl.forward(None, out.clone(), t(k, dev), t(v, dev), kv_cache, md, output=out)
    cache = impl_cls._tq_gpu_cache
    assert cache is not None and cache.max_blocks == NB and torch.all(kv_cache == 0)
    cache.tq.rotation = torch.from_numpy(R).to(dev)
    # layer 0 ran before the copy's rotation was replaced: rewrite both layers with the pinned matrix
    for li in range(LAYERS):
        cache.encode_and_store(li, t(k, dev), t(v, dev), md.slot_mapping)
    kd, vd = kv_like(rng, (1, KVH, 128)), kv_like(rng, (1, KVH, 128))
    qd = rng.standard_normal((1, QH, 128)).astype(np.float16)
    mdd = meta(dev, slots_of(tables, 0, 20, 21), tables, [21], 1, 1)
    outd = torch.zeros(1, QH * 128, dtype=torch.float16, device=dev)
    layers[1].forward(None, t(qd, dev).view(1, -1), t(kd, dev), t(vd, dev), kv_cache, mdd, output=outd)
    ref = O.paged_attention(qd, cache.k_packed[1].cpu().numpy(), cache.k_norms[1].cpu().numpy(),
                            cache.v_packed[1].cpu().numpy(), cache.v_norms[1].cpu().numpy(), tables, np.array([21]),
                            R, cen, 4, block_size=BS, dtype=np.float64, cast_output=False)
    assert within_tol(outd.view(1, QH, 128).cpu().numpy(), ref)
    assert float(cache.k_norms[1][3, 4, 0]) > 0 and float(cache.k_norms[0][3, 4, 0]) == 0     # token 20 -> block 3, row 4


def test_profiling_run_and_draft_layers(dev, impl_cls):
    target = impl_cls(QH, 128, 0.1, num_kv_heads=KVH, kv_cache_dtype="tq-t4nc")
    draft = impl_cls(4, 64, 0.1, num_kv_heads=1, kv_cache_dtype="tq-t4nc")
    assert target._tq_layer_idx == 0 and draft._is_draft and draft._tq_layer_idx == -1 and impl_cls._tq_layer_counter == 1
    out = torch.ones(3, QH * 128, dtype=torch.float16, device=dev)
    assert target.forward(None, out.clone(), None, None, torch.empty(0), None, output=out) is out and torch.all(out == 0)
    kv = torch.zeros(2, 2, BS, 1, 36, dtype=torch.uint8, device=dev)
    draft.do_kv_cache_update(None, torch.zeros(1, 1, 64, device=dev), torch.zeros(1, 1, 64, device=dev), kv,
                             torch.zeros(1, dtype=torch.int64, device=dev))
    assert torch.all(kv == 0)
    with pytest.raises(RuntimeError, match="vLLM"):
        draft.forward(None, out, None, None, kv, types.SimpleNamespace(max_query_len=1), output=out)

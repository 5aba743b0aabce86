"""Host-side behaviour that needs no GPU: configuration errors, sizes and layouts, init-time
tables against the reference's, the C-ABI library's exports, and the loud failure on CPU
tensors (reference: tests/test_core.py:246-425, tests/test_hybrid_hooks.py:411-442,
tests/test_triattention.py:62-86)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import aitherkvcache_amd as akv
from aitherkvcache_amd import _lib
from aitherkvcache_amd.codebook import get_codebook, get_theory_bounds
from aitherkvcache_amd.hybrid_quantizer import (HybridTurboQuant, _make_hybrid_layout,
                                                _lloyd_on_grid, dimension_aware_codebook)
from aitherkvcache_amd.packing import packed_size
from aitherkvcache_amd.rotation import (random_orthogonal, hadamard_matrix, random_signs,
                                        randomized_hadamard_matrix, fast_hadamard_transform)
from aitherkvcache_amd.triattention import TriAttentionConfig, TriAttention, rope_frequencies
from aitherkvcache_amd.vllm import resolve_kv_cache_dtype, register_custom_ops
from aitherkvcache_amd.vllm.kv_cache_dtype import tq_dim_for_head

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- the C ABI -----------------------------------------------------------------------------
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "aitherkv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(akv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 18
    assert os.path.exists(_lib.LIB_PATH), "build the HIP library first (make -C aitherkvcache_amd/csrc)"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in names if not hasattr(handle, n)]
    assert not missing, missing
    # and the Python binding lists the same set
    assert sorted(_lib.SIGNATURES) == names


def test_library_loads_and_reports_version():
    L = _lib.lib()
    assert b"aitherkv" in L.akv_version()
    assert L.akv_rotation_prepared_bytes(128) >= 4 * 128 * 128 * 4      # four d x d float32 planes + tables
    # argument validation happens before any device work
    rc = L.akv_encode(None, 0, -1, 128, 128, None, None, 4, None, 64, None, None)
    assert rc == _lib.AKV_ERR_INVALID and b"akv_encode" in L.akv_last_error()
    rc = L.akv_encode(None, 0, 4, 96, 96, None, None, 4, None, 48, None, None)
    assert rc == _lib.AKV_ERR_UNSUPPORTED
    with pytest.raises(NotImplementedError):
        _lib.check(rc)
    with pytest.raises(ValueError):
        _lib.check(_lib.AKV_ERR_INVALID)
    # the tq25 entry points check like their tq35 counterparts: sizes, null pointers, rows shorter than 44 bytes
    assert L.akv_hybrid25_encode(None, 0, 0, 128, None, None, 44, None) == _lib.AKV_OK
    assert L.akv_hybrid25_encode(None, 0, -1, 128, None, None, 44, None) == _lib.AKV_ERR_INVALID
    assert L.akv_hybrid25_encode(None, 0, 3, 128, None, None, 44, None) == _lib.AKV_ERR_INVALID
    assert b"akv_hybrid25_encode" in L.akv_last_error()
    buf = (ctypes.c_char * 4096)()
    ptr = ctypes.addressof(buf)
    assert L.akv_hybrid25_encode(ptr, 0, 3, 128, ptr, ptr, 43, None) == _lib.AKV_ERR_INVALID
    assert L.akv_hybrid25_decode(ptr, 40, 3, ptr, ptr, 128, None) == _lib.AKV_ERR_INVALID
    assert L.akv_hybrid25_decode(None, 44, 0, None, None, 128, None) == _lib.AKV_OK


# ---- TurboQuant surface -------------------------------------------------------------------
def test_config_errors():
    with pytest.raises(ValueError, match="Supported bit-widths"):
        akv.TurboQuant(head_dim=128, bits=5, device="cpu")
    with pytest.raises(ValueError, match="power of 2"):
        akv.TurboQuant(head_dim=100, bits=4, device="cpu")


@pytest.mark.parametrize("bits,packed,ratio", [(4, 64, 3.8), (3, 48, 4.9), (2, 32, 7.1)])
def test_sizes_and_ratios(bits, packed, ratio):
    tq = akv.TurboQuant(head_dim=128, bits=bits, device="cpu")
    assert tq._packed_dim == packed == packed_size(128, bits)
    assert abs(tq.compression_ratio() - ratio) < 0.06
    assert tq.num_levels == 1 << bits
    assert tq.centroids.dtype == torch.float32 and tq.centroids.numel() == 1 << bits
    assert tq.boundaries_inner.numel() == (1 << bits) - 1
    assert "TurboQuant" in repr(tq) and f"bits={bits}" in repr(tq)
    rep = tq.memory_report(seq_len=1024)
    assert rep["ratio_vs_fp16"] == pytest.approx(256 / (packed + 4))
    assert (tq.theory_lower, tq.theory_upper) == get_theory_bounds(bits)


def test_cpu_tensors_fail_loudly():
    tq = akv.TurboQuant(head_dim=128, bits=4, device="cpu")
    with pytest.raises(RuntimeError, match="HIP devices only"):
        tq.encode(torch.zeros(2, 128))
    with pytest.raises(RuntimeError, match="HIP devices only"):
        tq.decode(torch.zeros(2, 64, dtype=torch.uint8), torch.zeros(2))
    with pytest.raises(RuntimeError, match="HIP devices only"):
        akv.fused_tq4_kv_update(torch.zeros(1, 1, 128), torch.zeros(1, dtype=torch.int64),
                                torch.zeros(1, 16, 1, 64, dtype=torch.uint8), torch.zeros(1, 16, 1),
                                tq.rotation, tq.boundaries_inner)
    # an empty update returns before touching anything, like the reference (fused_kv_update.py:340)
    akv.fused_tq4_kv_update(torch.zeros(0, 1, 128), torch.zeros(0, dtype=torch.int64),
                            torch.zeros(1, 16, 1, 64, dtype=torch.uint8), torch.zeros(1, 16, 1),
                            tq.rotation, tq.boundaries_inner)
    with pytest.raises(ValueError, match="power of 2"):
        akv.fused_tq4_kv_update(torch.zeros(1, 1, 96), torch.zeros(1, dtype=torch.int64),
                                torch.zeros(1, 16, 1, 48, dtype=torch.uint8), torch.zeros(1, 16, 1),
                                tq.rotation, tq.boundaries_inner)


# ---- init-time tables against the reference ------------------------------------------------
def test_rotation_matches_reference(golden):
    for d in (64, 128):
        R = random_orthogonal(d, seed=42, device="cpu").numpy()
        assert R.dtype == np.float32
        # LAPACK's blocked QR rounds differently with the thread count, so the reference's own
        # matrix moves by ~1e-6 between runs on different machines
        assert np.max(np.abs(R - golden[f"rotation_d{d}_seed42"])) < 1e-5
        assert np.allclose(R @ R.T, np.eye(d), atol=1e-5)
    assert np.array_equal(random_orthogonal(128, 3, "cpu").numpy(), random_orthogonal(128, 3, "cpu").numpy())
    assert not np.allclose(random_orthogonal(128, 3, "cpu").numpy(), random_orthogonal(128, 4, "cpu").numpy())
    nthreads = torch.get_num_threads()
    try:
        torch.set_num_threads(1)
        assert np.array_equal(random_orthogonal(128, 42, "cpu").numpy(), golden["rotation_d128_seed42"])
    finally:
        torch.set_num_threads(nthreads)


def test_hadamard_helpers():
    H = hadamard_matrix(16)
    assert torch.allclose(H @ H.T, torch.eye(16), atol=1e-6)
    x = torch.randn(3, 16)
    assert torch.allclose(fast_hadamard_transform(x), x @ (H * 4).T, atol=1e-5)
    M = randomized_hadamard_matrix(32, device="cpu")
    assert torch.allclose(M @ M.T, torch.eye(32), atol=1e-5)
    s = random_signs(64, seed=1, device="cpu")
    assert set(s.tolist()) <= {-1.0, 1.0} and torch.equal(s, random_signs(64, seed=1, device="cpu"))
    with pytest.raises(AssertionError):
        hadamard_matrix(12)


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_codebook_matches_reference(golden, bits):
    c, b, _ = get_codebook(128, bits)
    assert np.array_equal(c.astype(np.float32), golden[f"centroids_b{bits}"])
    assert np.array_equal(b.astype(np.float32), golden[f"boundaries_b{bits}"])
    with pytest.raises(ValueError):
        get_codebook(128, 5)


def test_hybrid_host_state_matches_reference(golden):
    h = HybridTurboQuant(head_dim=128, mode="tq35", seed=42, device="cpu")
    for nm in ("g0_had", "g1_had", "g0_qjl", "g1_qjl"):
        assert np.array_equal(getattr(h, f"_{nm}_signs").numpy(), golden[f"hyb_{nm}_signs"])
    for g, bits in ((0, 3), (1, 2)):
        assert np.array_equal(getattr(h, f"_g{g}_centroids").numpy(), golden[f"hyb_centroids_64_{bits}"])
        assert np.array_equal(getattr(h, f"_g{g}_boundaries").numpy(), golden[f"hyb_boundaries_64_{bits}"])
        # and the general routine reproduces the tabulated case up to the noise in the middle boundary
        c, b = _lloyd_on_grid(64, bits)
        assert np.array_equal(c, golden[f"hyb_centroids_64_{bits}"])
        assert np.allclose(b, golden[f"hyb_boundaries_64_{bits}"], rtol=0, atol=1e-15)
    tab = h._table.numpy()
    assert tab.shape == (_lib.HYB_TABLE_FLOATS,)
    assert np.array_equal(tab[128:192], golden["hyb_g0_qjl_signs"])
    assert np.array_equal(tab[256:264], golden["hyb_centroids_64_3"])
    assert np.array_equal(tab[275:278], golden["hyb_boundaries_64_2"])
    c, b = dimension_aware_codebook(32, 2)
    assert c.numel() == 4 and torch.all(c[1:] > c[:-1])


def test_hybrid_layout_and_errors():
    lay = _make_hybrid_layout(128, "tq35")
    assert (lay.group0.total_bytes, lay.group1.total_bytes, lay.packed_dim) == (36, 28, 64)
    assert HybridTurboQuant.packed_dim_for_mode(128, "tq35") == 64
    assert HybridTurboQuant.packed_dim_for_mode(128, "tq25") == 8 + 4 + 4 + 12 + 12 + 4
    with pytest.raises(ValueError, match="Unsupported mode"):
        HybridTurboQuant(mode="tq99", device="cpu")
    h = HybridTurboQuant(device="cpu")
    with pytest.raises(RuntimeError, match="calibrate"):
        h.encode(torch.zeros(1, 128))
    h.calibrate_uniform(num_kv_heads=8)
    assert h._group0_indices.shape == (8, 64) and int(h._group1_indices[0, 0]) == 64
    with pytest.raises(RuntimeError, match="HIP devices only"):
        h.encode(torch.zeros(1, 128))
    assert h.compression_ratio() == 4.0 and "calibrated" in repr(h)
    with pytest.raises(NotImplementedError, match="head_dim 128 only"):
        h64 = HybridTurboQuant(head_dim=64, device="cpu")
        h64.calibrate_uniform()
        h64.encode(torch.zeros(1, 64))


def test_tq25_constants_match_the_reference(tq25):
    """Mode tq25 on the host: the sign vectors of seed 42, the two codebooks (literal tables: the one-bit
    book's boundary is float64 summation noise in the reference) and the kernel table's layout."""
    t = HybridTurboQuant(mode="tq25", device="cpu")
    assert (t._g0_dim, t._g1_dim, t._g0_mse_bits, t._g1_mse_bits, t.packed_dim) == (32, 96, 2, 1, 44)
    for nm, got in (("g0_had", t._g0_had_signs), ("g1_had", t._g1_had_signs), ("g0_qjl", t._g0_qjl_signs),
                    ("g1_qjl", t._g1_qjl_signs), ("g0_centroids", t._g0_centroids), ("g0_boundaries", t._g0_boundaries),
                    ("g1_centroids", t._g1_centroids), ("g1_boundaries", t._g1_boundaries)):
        assert np.array_equal(got.numpy(), tq25[nm]), nm
    tab = t._table.numpy()
    assert tab.shape == (_lib.HYB_TABLE_FLOATS,)
    assert np.array_equal(tab[0:32], tq25["g0_had"]) and np.array_equal(tab[32:128], tq25["g1_had"])
    assert np.array_equal(tab[128:160], tq25["g0_qjl"]) and np.array_equal(tab[160:256], tq25["g1_qjl"])
    assert np.array_equal(tab[256:260], tq25["g0_centroids"]) and np.array_equal(tab[260:262], tq25["g1_centroids"])
    assert np.array_equal(tab[262:265], tq25["g0_boundaries"]) and np.array_equal(tab[265:266], tq25["g1_boundaries"])
    assert t._abi == "akv_hybrid25" and HybridTurboQuant(device="cpu")._abi == "akv_hybrid"
    t.calibrate_uniform(num_kv_heads=2)
    assert t._group0_indices.shape == (2, 32) and int(t._group1_indices[1, 0]) == 32
    with pytest.raises(RuntimeError, match="HIP devices only"):
        t.encode(torch.zeros(1, 128))
    # the grid iteration itself gives the same centroids as the literal tables
    from aitherkvcache_amd.hybrid_quantizer import _lloyd_on_grid
    for (d, b), nm in (((32, 2), "g0"), ((96, 1), "g1")):
        assert np.array_equal(_lloyd_on_grid(d, b)[0], tq25[nm + "_centroids"])


def test_tri_config_and_theta(golden):
    c = TriAttentionConfig()
    assert c.bytes_per_kv_token == 26 and c.fp16_bytes_per_kv_token == 256 and c.compression_ratio > 9
    assert TriAttentionConfig(coeff_bits=8).bytes_per_kv_token == 38
    assert TriAttentionConfig(coeff_bits=16).bytes_per_kv_token == 62
    with pytest.raises(ValueError, match="head_dim must be even"):
        TriAttentionConfig(head_dim=127)
    with pytest.raises(ValueError, match="cannot exceed"):
        TriAttentionConfig(head_dim=32, num_freqs=20)
    with pytest.raises(ValueError, match="coeff_bits"):
        TriAttentionConfig(coeff_bits=6)
    assert TriAttentionConfig(num_freqs=10, layer_freq_schedule=[16, 14]).freq_budget(1) == 14
    assert np.array_equal(rope_frequencies(128, 1e6).numpy(), golden["theta_d128_base1e6"])
    assert np.array_equal(rope_frequencies(32, 1e4).numpy(), golden["theta_d32_base1e4"])
    tri = TriAttention(c, device="cpu")
    enc = tri.encoder.encode(torch.from_numpy(golden["tri_keys"].astype(np.float32)))
    assert np.array_equal(enc.indices.numpy(), golden["tri_k_indices"])
    assert np.array_equal(enc.packed.numpy(), golden["tri_k_packed"])
    assert np.array_equal(enc.scales.numpy(), golden["tri_k_scales"])


def test_kv_cache_dtype_names_and_ops():
    assert resolve_kv_cache_dtype("tq-t4nc").bits == 4
    assert resolve_kv_cache_dtype("TQ-T3NC").bits == 3
    assert resolve_kv_cache_dtype("tq-t2nc").packed_bytes_d128 == 32
    assert resolve_kv_cache_dtype("tq35").mode == "tq35"
    assert tq_dim_for_head(128, resolve_kv_cache_dtype("tq-t4nc")) == 68
    assert tq_dim_for_head(128, resolve_kv_cache_dtype("tq-t35nc")) == 64
    assert resolve_kv_cache_dtype("tq25").mode == "tq25" and tq_dim_for_head(128, resolve_kv_cache_dtype("tq25")) == 44
    with pytest.raises(ValueError):
        resolve_kv_cache_dtype("fp8")
    assert register_custom_ops() and register_custom_ops()
    assert hasattr(torch.ops.tq, "decode_step") and hasattr(torch.ops.tq, "hybrid_decode_step")


def test_primary_cache_layout_arithmetic():
    """Page size, power-of-two page alignment and the PRIMARY uint8 layout
    (reference: aither_kvcache/vllm/engine.py:110-154, 340-375)."""
    from aitherkvcache_amd.vllm import tq_page_size_bytes, align_page_size, reshape_primary, primary_views
    f4, f3, fh = (resolve_kv_cache_dtype(n) for n in ("tq-t4nc", "tq-t3nc", "tq35"))
    assert tq_page_size_bytes(16, 8, 128, f4) == 2 * 16 * 8 * 68 == 17408
    assert tq_page_size_bytes(16, 8, 128, f3) == 2 * 16 * 8 * 52
    assert tq_page_size_bytes(16, 8, 128, fh) == 2 * 16 * 8 * 64 == 16384
    assert [align_page_size(v) for v in (0, -3, 1, 2, 3, 17408, 16384, 16385)] == [0, -3, 1, 2, 4, 32768, 16384, 32768]
    page = align_page_size(tq_page_size_bytes(16, 8, 128, f4))
    raw = torch.arange(3 * page, dtype=torch.int64).to(torch.uint8)      # three padded pages, as bytes
    kv = reshape_primary(raw, 3, 16, 8, 128, f4)
    assert kv.shape == (3, 2, 16, 8, 68) and kv.dtype == torch.uint8
    assert kv.data_ptr() == raw.data_ptr()                               # a view, nothing copied
    k, v = primary_views(kv, 128, f4)
    assert k.shape == v.shape == (3, 16, 8, 64)
    assert k.stride() == (2 * 16 * 8 * 68, 8 * 68, 68, 1)
    assert v.data_ptr() - k.data_ptr() == 16 * 8 * 68
    assert int(k[1, 2, 3, 5]) == (1 * 2 * 16 * 8 * 68 + (2 * 8 + 3) * 68 + 5) % 256
    with pytest.raises(ValueError):
        reshape_primary(raw[:100], 3, 16, 8, 128, f4)
    with pytest.raises(ValueError):
        primary_views(kv, 128, fh)
    kh = reshape_primary(torch.zeros(2 * 16384, dtype=torch.uint8), 2, 16, 8, 128, fh)
    a, b = primary_views(kh, 128, fh)
    assert a.shape == (2, 16, 8, 64) and b.stride(2) == 64


def test_spectral_kv_cache_bookkeeping():
    """SpectralKVCache on the CPU: store / fetch round trips, copy, clear, statistics
    (reference: tests/test_triattention.py:225-247, 460-473; triattention/cache.py)."""
    from aitherkvcache_amd.triattention import SpectralKVCache, SpectralEncoding
    from oracle import tq_oracle as O
    cfg = TriAttentionConfig(num_kv_heads=2, num_query_heads=8)
    cache = SpectralKVCache(cfg, max_blocks=6)
    BS, KVH, F = cfg.block_size, 2, cfg.num_freqs
    g = torch.Generator().manual_seed(5)

    def enc(n):
        return SpectralEncoding(torch.randint(0, 64, (n, KVH, F), dtype=torch.uint8, generator=g),
                                torch.randint(0, 256, (n, KVH, F), dtype=torch.uint8, generator=g),
                                torch.rand(n, KVH, generator=g).half())

    S = 2 * BS + 5
    k, v = enc(S), enc(S)
    table = torch.tensor([4, 1, 3, 0])
    cache.store_block(4, SpectralEncoding(*(x[:BS] for x in k)), SpectralEncoding(*(x[:BS] for x in v)))
    cache.store_block(1, SpectralEncoding(*(x[BS:2 * BS] for x in k)), SpectralEncoding(*(x[BS:2 * BS] for x in v)))
    for j in range(5):
        tok = 2 * BS + j
        cache.store_token(3, j, SpectralEncoding(*(x[tok] for x in k)), SpectralEncoding(*(x[tok] for x in v)))
    k_out, v_out = cache.fetch_sequence(table, S)
    for a, b in zip(tuple(k_out) + tuple(v_out), tuple(k) + tuple(v)):
        assert torch.equal(a, b)
    ko, vo = O.spectral_fetch_sequence([x.numpy() for x in cache._arrays()], table.numpy(), S, BS)
    for a, b in zip(ko + vo, tuple(k) + tuple(v)):
        assert np.array_equal(a, b.numpy())
    stats = cache.memory_stats()
    assert stats["used_blocks"] == 3 and stats["total_tokens"] == S
    assert stats["bytes_allocated"] == 6 * BS * KVH * (F + F + 2) * 2 and cache.bytes_per_token == 52
    cache.copy_block(3, 5)
    assert torch.equal(cache.k_packed[5], cache.k_packed[3]) and cache.memory_stats()["total_tokens"] == S + 5
    cache.clear_block(4)
    assert int(cache.k_indices[4].sum()) == 0 and cache.memory_stats()["used_blocks"] == 3
    other = SpectralKVCache(cfg, max_blocks=6)
    other.store_sequence(table, k, v)
    k2, v2 = other.fetch_sequence(table, S)
    assert all(torch.equal(a, b) for a, b in zip(tuple(k2) + tuple(v2), tuple(k) + tuple(v)))
    assert other.memory_stats()["total_tokens"] == S


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_packing_helpers_match_the_pinned_layouts(bits):
    """pack_* / unpack_* of the public packing module against the oracle's restatement (itself pinned
    exhaustively over all bytes / all 2^24 three-bit words): random indices in several shapes, the
    round trip, and the reference's divisibility asserts."""
    import torch
    from aitherkvcache_amd import packing as P
    from oracle import tq_oracle as O
    rng = np.random.default_rng(bits)
    pack = {2: P.pack_2bit, 3: P.pack_3bit, 4: P.pack_4bit}[bits]
    unpack = {2: P.unpack_2bit, 3: P.unpack_3bit, 4: P.unpack_4bit}[bits]
    opack = {2: O.pack_2bit, 3: O.pack_3bit, 4: O.pack_4bit}[bits]
    for shape in ((128,), (5, 64), (2, 3, 128), (0, 128), (7, 8)):
        idx = rng.integers(0, 1 << bits, size=shape).astype(np.uint8)
        got = pack(torch.from_numpy(idx))
        assert got.dtype == torch.uint8 and got.shape[-1] == P.packed_size(shape[-1], bits)
        assert np.array_equal(got.numpy(), opack(idx))
        back = unpack(got, shape[-1])
        assert back.dtype == torch.uint8 and np.array_equal(back.numpy(), idx)
        assert np.array_equal(pack(torch.from_numpy(idx.astype(np.int64))).numpy(), got.numpy())   # any integer dtype
    with pytest.raises(AssertionError):
        pack(torch.zeros(1, {2: 6, 3: 12, 4: 7}[bits], dtype=torch.uint8))


def test_backend_module_needs_no_vllm_and_no_gpu():
    """Importing the backend module and making its classes imports no vLLM; the class answers vLLM's
    questions (reference: vllm/backend.py:264-311) and the plugin entry point reports that there is
    nothing to register with (vllm/plugin.py:18-53)."""
    import sys
    from aitherkvcache_amd.vllm import backend, plugin
    bk = backend.TurboQuantBackend
    assert not any(m == "vllm" or m.startswith("vllm.") for m in sys.modules)
    assert bk.get_name() == "CUSTOM" and bk.accept_output_buffer is True
    assert bk.forward_includes_kv_cache_update is False
    assert bk.get_kv_cache_shape(9, 16, 8, 128) == (9, 2, 16, 8, 128)
    assert bk.get_kv_cache_shape(9, 16, 8, 128, "fp8") == (9, 2, 16, 8, 128)
    assert bk.get_kv_cache_shape(9, 16, 8, 128, "tq-t4nc") == (9, 2, 16, 8, 68)
    assert bk.get_kv_cache_shape(9, 16, 8, 128, "tq-t3nc") == (9, 2, 16, 8, 52)
    assert bk.get_kv_cache_shape(9, 16, 8, 128, "tq-t2nc") == (9, 2, 16, 8, 36)
    assert bk.get_kv_cache_shape(9, 16, 8, 128, "tq35") == (9, 2, 16, 8, 64)
    assert bk.get_supported_head_sizes() == [64, 96, 128, 256, 512]
    assert {"auto", "bfloat16", "fp8", "tq-t4nc", "tq-t3nc", "tq-t2nc", "tq35"} <= set(bk.supported_kv_cache_dtypes)
    impl = bk.get_impl_cls()
    assert impl is backend.TurboQuantImpl and callable(impl.do_kv_cache_update) and callable(impl.forward)
    assert backend.register_turboquant_backend() is False and plugin.register() is False
    with pytest.raises(AttributeError):
        backend.NoSuchName


def test_backend_format_selection_from_environment(monkeypatch):
    from aitherkvcache_amd.vllm import backend
    for mode, bits_env, want in (("", None, ("uniform", 4)), ("", "3", ("uniform", 3)), ("tq35", None, ("hybrid", None)),
                                 ("tq35-primary", None, ("hybrid", None)), ("tq-t2nc-primary", "4", ("uniform", 2))):
        monkeypatch.setenv("AITHER_TQ_MODE", mode)
        if bits_env is None:
            monkeypatch.delenv("AITHER_TQ_BITS", raising=False)
        else:
            monkeypatch.setenv("AITHER_TQ_BITS", bits_env)
        fmt = backend.format_from_env()
        assert (fmt.kind, fmt.bits) == want
        assert backend.primary_from_env() == mode.endswith("-primary")
    monkeypatch.setenv("AITHER_TQ_MODE", "")
    monkeypatch.setenv("AITHER_TQ_PRIMARY", "1")
    assert backend.primary_from_env()


def test_tri_helpers_on_host_tensors():
    """Spectral helpers, adaptive pair count and the dense RoPE attention helper are torch ops and run anywhere."""
    from oracle import tq_oracle as O
    from aitherkvcache_amd.triattention import SpectralKVEncoder, TriAttention, TriAttentionConfig
    from aitherkvcache_amd.triattention.spectral import pair_energies, pair_energy_profile, spectral_concentration, topk_pairs
    x = torch.tensor([[3.0, 4.0, 0.0, 1.0, 2.0, 0.0, 0.5, 0.5]])
    assert torch.equal(pair_energies(x), torch.tensor([[25.0, 1.0, 4.0, 0.5]]))
    idx, vals = topk_pairs(x, 2)
    assert idx.dtype == torch.uint8 and idx.tolist() == [[0, 2]] and vals.tolist() == [[[3.0, 4.0], [2.0, 0.0]]]
    assert abs(spectral_concentration(x, 2).item() - 29.0 / 30.5) < 1e-6
    assert pair_energy_profile(x).tolist() == [[25.0, 4.0, 1.0, 0.5]]
    cfg = TriAttentionConfig(head_dim=8, num_freqs=1, coeff_bits=16, num_kv_heads=1, num_query_heads=1, rope_base=1e4)
    enc = SpectralKVEncoder(cfg)
    e, needed = enc.encode_adaptive(x, min_energy_ratio=0.9)       # 25 / 30.5 < 0.9 <= 29 / 30.5
    assert needed.tolist() == [2] and e.indices.tolist() == [[0, 2]]
    st = enc.compression_stats(x)
    assert st["num_freqs"] == 1 and abs(st["energy_ratio"] - 25.0 / 30.5) < 1e-6 and abs(st["mse"] - 5.5 / 8) < 1e-6
    # dense RoPE attention against the oracle's dense attention on rotated tensors
    rng = np.random.default_rng(0)
    B, S, QH, KVH, D = 2, 9, 4, 2, 8
    q, k, v = rng.standard_normal((B, QH, D)), rng.standard_normal((B, S, KVH, D)), rng.standard_normal((B, S, KVH, D))
    got = TriAttention.reference_attention(torch.from_numpy(q).float(), torch.from_numpy(k).float(),
                                           torch.from_numpy(v).float(), 1e4).numpy()
    theta = O.rope_frequencies(D, 1e4).astype(np.float64)

    def rope(x, pos):
        ang = pos[..., None] * theta
        xe, xo = x[..., 0::2], x[..., 1::2]
        return np.stack((xe * np.cos(ang) - xo * np.sin(ang), xe * np.sin(ang) + xo * np.cos(ang)), -1).reshape(x.shape)

    qr = rope(q, np.full((B, 1), float(S)))
    kr = rope(k, np.broadcast_to(np.arange(S, dtype=np.float64)[None, :, None], (B, S, 1)))
    for b in range(B):
        for h in range(QH):
            s = kr[b, :, h // 2] @ qr[b, h] / np.sqrt(D)
            w = np.exp(s - s.max()); w /= w.sum()
            assert np.max(np.abs(got[b, h] - w @ v[b, :, h // 2])) < 1e-5


def test_hybrid_module_helpers_against_the_oracle():
    """fwht_pow2 / fwht_general / structured_hadamard / pack_multibit / unpack_multibit of the public module."""
    from oracle import tq_oracle as O
    from aitherkvcache_amd.hybrid_quantizer import (fwht_general, fwht_pow2, pack_multibit, structured_hadamard,
                                                    unpack_multibit)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 64)).astype(np.float32)
    xt = torch.from_numpy(x.copy())
    assert fwht_pow2(xt) is xt and np.allclose(xt.numpy(), O.fwht(x), rtol=1e-6, atol=1e-5)
    # H H = N I: a second call on the SAME tensor must transform it again (nothing is cached per argument)
    assert fwht_pow2(xt) is xt and np.allclose(xt.numpy(), 64.0 * x, rtol=1e-5, atol=1e-4)
    ones = torch.ones(4)
    assert fwht_pow2(ones).tolist() == [4.0, 0.0, 0.0, 0.0] and fwht_pow2(ones).tolist() == [4.0, 4.0, 4.0, 4.0]
    assert not hasattr(fwht_pow2, "cache_info")
    y = rng.standard_normal((3, 96)).astype(np.float32)
    got = fwht_general(torch.from_numpy(y)).numpy()
    assert np.allclose(got[:, :64], O.fwht(y[:, :64]), atol=1e-5) and np.allclose(got[:, 64:], O.fwht(y[:, 64:]), atol=1e-5)
    signs = np.where(rng.integers(0, 2, 64) > 0, 1.0, -1.0).astype(np.float32)
    fwd = structured_hadamard(torch.from_numpy(x), torch.from_numpy(signs))
    assert np.allclose(fwd.numpy(), O.structured_hadamard(x, signs), atol=1e-5)
    back = structured_hadamard(fwd, torch.from_numpy(signs), inverse=True)
    assert np.allclose(back.numpy(), x, atol=1e-5)
    for bits, dim in ((1, 64), (2, 64), (3, 64), (4, 30), (3, 7)):
        idx = rng.integers(0, 1 << bits, size=(4, dim)).astype(np.uint8)
        p = pack_multibit(torch.from_numpy(idx), bits)
        assert p.dtype == torch.uint8 and np.array_equal(p.numpy(), O.pack_multibit(idx, bits))
        assert np.array_equal(unpack_multibit(p, dim, bits).numpy(), idx)


def test_codebook_from_the_density_reproduces_the_tables():
    from aitherkvcache_amd.codebook import compute_codebook_scipy
    cen, bnd, mse = compute_codebook_scipy(128, 2, max_iter=200, tol=1e-10)
    ref_c, ref_b, ref_mse = get_codebook(128, 2)
    assert np.allclose(cen, ref_c, atol=1e-5) and np.allclose(bnd, ref_b, atol=1e-5) and abs(mse - ref_mse) < 2e-4   # (support cut at 5 sigma)
    assert "GQA 4:1" in akv.triattention.TriAttentionConfig().summary()


def test_ranked_calibration_orders_coordinates_by_mean_square():
    """HybridTurboQuant.calibrate: per kv head the 64 coordinates of largest mean square first, in descending order,
    then the rest; to_group_order / from_group_order are inverse gathers with the reference's head rules."""
    h = HybridTurboQuant(device="cpu")
    rng = np.random.default_rng(7)
    scale = rng.permutation(128).astype(np.float32) + 1.0                       # distinct scores
    sample = torch.from_numpy(np.stack([np.ones((50, 128), np.float32) * scale,
                                        np.ones((50, 128), np.float32) * scale[::-1]], axis=1))   # [50, 2, 128]
    with pytest.raises(ValueError):
        h.calibrate(sample[0])
    h.calibrate(sample)
    want0 = np.argsort(-scale, kind="stable")
    assert h._group0_indices.shape == (2, 64) and h._group1_indices.shape == (2, 64)
    assert np.array_equal(h._group0_indices[0].numpy(), want0[:64]) and np.array_equal(h._group1_indices[0].numpy(), want0[64:])
    assert np.array_equal(h.group_order[1].numpy(), np.argsort(-scale[::-1], kind="stable"))
    x = torch.from_numpy(rng.standard_normal((6, 2, 128)).astype(np.float32))
    g = h.to_group_order(x, head_axis=1)
    assert torch.equal(g[:, 0], x[:, 0][:, h.group_order[0]]) and torch.equal(g[:, 1], x[:, 1][:, h.group_order[1]])
    assert torch.equal(h.from_group_order(g, head_axis=1), x)
    # without a head axis: vectors cycle over the heads when their number is a multiple of the head count ...
    assert torch.equal(h.to_group_order(x.reshape(12, 128)), g.reshape(12, 128))
    # ... and use head 0's order otherwise
    odd = x.reshape(12, 128)[:3]
    assert torch.equal(h.to_group_order(odd), odd[:, h.group_order[0]])
    assert torch.equal(h.from_group_order(h.to_group_order(odd)), odd)
    u = HybridTurboQuant(device="cpu")
    u.calibrate_uniform(4)
    assert u.group_order is None and u.to_group_order(x) is x


def test_tri_pair_series_and_dct_helpers():
    """The pairwise series equals the dot product of explicitly rotated vectors (the identity the scorer rests on);
    the DCT matrix is orthogonal, equals scipy's orthonormal DCT-II and inverts."""
    import scipy.fft
    from aitherkvcache_amd.triattention.spectral import (dct, dct_matrix, idct, rope_frequencies, rope_phase_matrix,
                                                           trig_series_coefficients)
    rng = np.random.default_rng(5)
    B, S, D = 2, 7, 16
    q = torch.from_numpy(rng.standard_normal((B, 1, D)))
    k = torch.from_numpy(rng.standard_normal((B, S, D)))
    theta = rope_frequencies(D, 1e4, dtype=torch.float64)
    qpos = torch.tensor([11, 3]); kpos = torch.from_numpy(rng.integers(0, 20, size=(B, S)))
    c, s_ = trig_series_coefficients(q.expand(B, S, D), k)
    cp, sp = rope_phase_matrix(qpos, kpos, theta)
    series = (c * cp + s_ * sp).sum(-1)

    def rope(x, pos):
        ang = pos.double().unsqueeze(-1) * theta
        xe, xo = x[..., 0::2], x[..., 1::2]
        return torch.stack((xe * torch.cos(ang) - xo * torch.sin(ang), xe * torch.sin(ang) + xo * torch.cos(ang)), -1).flatten(-2)
    direct = (rope(q, qpos.view(B, 1)) * rope(k, kpos)).sum(-1)
    assert float((series - direct).abs().max()) < 1e-12
    idx = torch.tensor([1, 6]).expand(B, S, 2)
    c2, s2 = trig_series_coefficients(q.expand(B, S, D), k, idx)
    assert torch.equal(c2, c[..., [1, 6]]) and torch.equal(s2, s_[..., [1, 6]])
    Dm = dct_matrix(12, dtype=torch.float64)
    assert float((Dm @ Dm.T - torch.eye(12, dtype=torch.float64)).abs().max()) < 1e-14
    x = torch.from_numpy(rng.standard_normal((3, 12)))
    assert np.max(np.abs(dct(x).numpy() - scipy.fft.dct(x.numpy(), type=2, norm="ortho", axis=-1))) < 1e-13
    assert float((idct(dct(x, Dm), Dm) - x).abs().max()) < 1e-13


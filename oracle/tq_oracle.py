"""CPU oracle for the TurboQuant / tq35 and tq25 / TriAttention hot path  --  TEST INFRASTRUCTURE ONLY.

This module is a plain numpy restatement of the reference's algorithm for the
path (encode-on-write -> paged decode attention -> TriAttention decode_step).
It exists to CHECK the HIP kernels.  Nothing in the shipped package imports it:
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may.

Every function cites the reference lines it restates (paths are relative to the
reference tree).  How each one is pinned:

  pinned by the committed golden vectors (tests/golden/golden_v1.npz, produced
  by running the reference itself) and by independent brute force / closed forms
  in tests/test_oracle_*.py:
      get_codebook, pack_*/unpack_*, pack_multibit/unpack_multibit,
      encode, decode, kv_update, paged_attention_loop, paged_attention,
      block_rep_update, block_rep_finalize, block_scores, block_select (golden vectors in
      tests/golden/golden_block_selector.npz, written by the reference itself),
      batch_decompress_active_blocks (its decode by the golden vectors; its block
      selection and scatter by a per-block loop in tests/test_oracle_pins.py),
      fwht, structured_hadamard, dimension_aware_codebook,
      hybrid_encode, hybrid_decode (mode tq25, with fwht_general over 96 points, by
      tests/golden/golden_tq25.npz, also written by the reference itself, and by the block
      structure of the 96-point matrix), rope_frequencies, spectral_encode,
      tri_scores, tri_decode_step (coefficient widths 8 / 16 and post-RoPE scoring by
      tests/golden/golden_tri_widths.npz, also written by the reference itself),
      spectral_fetch_sequence / tri_decode_step_paged (indexing only, on top of the pinned
      tri_decode_step: checked against a token-by-token loop in tests/test_oracle_pins.py)
  derived here (the reference has no such function; it always decompresses
  tq35 / tq25 data before attending): hybrid_paged_attention is *defined* as
  hybrid_decode -> dense f32 softmax attention, i.e. the reference's
  tq::hybrid_decode_step (vllm/hooks.py:294-345) without its bf16 down-cast.

Inputs that only torch's CPU generator / LAPACK can produce (the rotation matrix
and the tq35 / tq25 sign vectors) are arguments here; the tests take them from the
golden file.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np

f32 = np.float32

# --------------------------------------------------------------------------------------
# codebook.py
# --------------------------------------------------------------------------------------
# Lloyd-Max centroids of N(0,1) (Max 1960), as tabulated at codebook.py:28-53.
_STD_CENTROIDS = {
    1: [-0.798284, 0.798284],
    2: [-1.510469, -0.452781, 0.452781, 1.510469],
    3: [-2.152090, -1.344134, -0.756031, -0.245104, 0.245104, 0.756031, 1.344134, 2.152090],
    4: [-2.733266, -2.069016, -1.618002, -1.256233, -0.942391, -0.656804, -0.388089, -0.128350,
        0.128350, 0.388089, 0.656804, 0.942391, 1.256233, 1.618002, 2.069016, 2.733266],
}
_STD_MSE = {1: 0.363480, 2: 0.117517, 3: 0.034506, 4: 0.009497}


def get_codebook(d: int, bits: int):
    """codebook.py:62-82 + quantizer.py:96-99: centroids/sqrt(d) in float64, boundaries are
    midpoints, both cast to float32 by the quantizer."""
    if bits not in _STD_CENTROIDS:
        raise ValueError(f"Supported bit-widths: {list(_STD_CENTROIDS)}. Got {bits}")
    c = np.array(_STD_CENTROIDS[bits], dtype=np.float64) * (1.0 / math.sqrt(d))
    b = (c[:-1] + c[1:]) / 2
    return c.astype(f32), b.astype(f32), _STD_MSE[bits]


def theory_bounds(bits: int):
    """codebook.py:85-89."""
    return 1.0 / 4 ** bits, (3 * math.pi / 2) / 4 ** bits


# --------------------------------------------------------------------------------------
# packing.py
# --------------------------------------------------------------------------------------
def packed_size(dim: int, bits: int) -> int:
    """packing.py:121-131."""
    if bits == 4:
        return dim // 2
    if bits == 3:
        assert dim % 8 == 0
        return dim * 3 // 8
    if bits == 2:
        return dim // 4
    raise ValueError(f"Unsupported bit-width: {bits}")


def pack_4bit(idx):
    """packing.py:13-23: byte k = idx[2k] << 4 | idx[2k+1]."""
    idx = np.asarray(idx).astype(np.uint8)
    return ((idx[..., 0::2] << 4) | idx[..., 1::2]).astype(np.uint8)


def unpack_4bit(packed, dim):
    """packing.py:26-37."""
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.empty(packed.shape[:-1] + (dim,), dtype=np.uint8)
    out[..., 0::2] = (packed >> 4) & 0x0F
    out[..., 1::2] = packed & 0x0F
    return out


def pack_2bit(idx):
    """packing.py:40-52: byte k = a<<6 | b<<4 | c<<2 | d for idx[4k..4k+3]."""
    idx = np.asarray(idx).astype(np.uint8)
    return ((idx[..., 0::4] << 6) | (idx[..., 1::4] << 4) | (idx[..., 2::4] << 2)
            | idx[..., 3::4]).astype(np.uint8)


def unpack_2bit(packed, dim):
    """packing.py:55-70."""
    packed = np.asarray(packed, dtype=np.uint8)
    out = np.empty(packed.shape[:-1] + (dim,), dtype=np.uint8)
    for k in range(4):
        out[..., k::4] = (packed >> (6 - 2 * k)) & 0x03
    return out


def pack_3bit(idx):
    """packing.py:73-98: 8 values -> one 24-bit big-endian word, value i at bits 23-3i..21-3i."""
    idx = np.asarray(idx).astype(np.int32)
    D = idx.shape[-1]
    assert D % 8 == 0
    g = idx.reshape(idx.shape[:-1] + (D // 8, 8))
    bits24 = np.zeros(g.shape[:-1], dtype=np.int32)
    for i in range(8):
        bits24 |= (g[..., i] & 0x7) << (21 - 3 * i)
    b = np.stack([(bits24 >> 16) & 0xFF, (bits24 >> 8) & 0xFF, bits24 & 0xFF], axis=-1)
    return b.astype(np.uint8).reshape(idx.shape[:-1] + (D // 8 * 3,))


def unpack_3bit(packed, dim):
    """packing.py:101-118."""
    packed = np.asarray(packed, dtype=np.uint8)
    g = packed.reshape(packed.shape[:-1] + (dim // 8, 3)).astype(np.int32)
    bits24 = (g[..., 0] << 16) | (g[..., 1] << 8) | g[..., 2]
    out = np.empty(g.shape[:-1] + (8,), dtype=np.uint8)
    for i in range(8):
        out[..., i] = (bits24 >> (21 - 3 * i)) & 0x7
    return out.reshape(packed.shape[:-1] + (dim,))


_PACK = {2: pack_2bit, 3: pack_3bit, 4: pack_4bit}
_UNPACK = {2: unpack_2bit, 3: unpack_3bit, 4: unpack_4bit}


# --------------------------------------------------------------------------------------
# quantizer.py
# --------------------------------------------------------------------------------------
def quantize(y, boundaries, bits):
    """quantizer.py:203-207: idx = clamp(searchsorted(bnd, y, right=False)) = #{b : b < y}."""
    idx = np.searchsorted(np.asarray(boundaries, dtype=f32), np.asarray(y, dtype=f32), side="left")
    return np.clip(idx, 0, (1 << bits) - 1)


def rotate_unit(x, rotation):
    """quantizer.py:140-150: norms, u = x/(n+1e-10), y = u @ R.T, all float32."""
    xf = np.ascontiguousarray(np.asarray(x).astype(f32)).reshape(-1, rotation.shape[0])
    norms = np.sqrt(np.sum(xf * xf, axis=-1, dtype=f32)).astype(f32)
    u = xf / (norms[:, None] + f32(1e-10))
    y = u @ np.ascontiguousarray(rotation.T)
    return y.astype(f32), norms


def rotate_unit_f64(x, rotation):
    """Same quantity as rotate_unit with the dot products carried in float64.  Used to tell a
    rounding-order difference (rotated value within a few float32 ulps of a decision
    boundary) from a real defect when two float32 implementations disagree on a code."""
    xf = np.asarray(x).astype(f32).reshape(-1, rotation.shape[0])
    norms = np.sqrt(np.sum(xf.astype(np.float64) ** 2, axis=-1))
    u = (xf / (norms.astype(f32)[:, None] + f32(1e-10))).astype(np.float64)
    return u @ rotation.astype(np.float64).T


def boundary_ulp_distance(y64, boundaries, floor=None):
    """Distance from each float64 rotated value to the nearest decision boundary, in float32 ulps.
    The ulp is taken at the largest of |boundary|, |value| and `floor`.  `floor` is the magnitude of
    the largest term of the dot product that made the value: a float32 dot product resolves nothing
    below one ulp of its largest term, so where the terms cancel (a value a few 1e-9 from the
    boundary at 0 out of terms of 1e-2) the value's own ulp says nothing about what float32
    arithmetic can decide."""
    b = np.asarray(boundaries, dtype=np.float64)
    d = np.abs(y64[..., None] - b)
    k = np.argmin(d, axis=-1)
    nearest = b[k]
    scale = np.maximum(np.abs(nearest), np.abs(y64))
    if floor is not None:
        scale = np.maximum(scale, np.asarray(floor, dtype=np.float64))
    ulp = np.spacing(np.maximum(scale, 1e-30).astype(f32)).astype(np.float64)
    return np.min(d, axis=-1) / ulp


def code_mismatch_report(codes_a, codes_b, y64, boundaries, unit64=None, R=None):
    """Where two code arrays differ, how far (in float32 ulps) the float64 rotated value is from
    the nearest decision boundary.  With the unit vectors and the matrix given, the ulp is not taken
    below that of the largest term R[j, i] * u[i] of the coordinate's dot product (cancellation).
    Returns (count, max_ulps, histogram dict)."""
    diff = np.argwhere(codes_a != codes_b)
    if len(diff) == 0:
        return 0, 0.0, {}
    rows, cols = diff.T
    floor = None
    if unit64 is not None and R is not None:
        floor = np.max(np.abs(np.asarray(R, dtype=np.float64)[cols] * unit64[rows]), axis=-1)
    ulps = boundary_ulp_distance(y64[rows, cols], boundaries, floor)
    steps = np.abs(codes_a.astype(np.int64) - codes_b.astype(np.int64))[tuple(diff.T)]
    hist = {"<=1": int((ulps <= 1).sum()), "<=4": int(((ulps > 1) & (ulps <= 4)).sum()),
            "<=16": int(((ulps > 4) & (ulps <= 16)).sum()), ">16": int((ulps > 16).sum()),
            "max_code_step": int(steps.max())}
    return len(diff), float(ulps.max()), hist


def encode_parity_report(packed, norms, x, rotation, bits):
    """Codes and norms of some encoder against encode() of this file on the same vectors: how many codes
    differ, the histogram of the distances (float32 ulps) of their float64 rotated values from the
    decision boundary, and the largest relative difference of the norms."""
    d = rotation.shape[0]
    _, b, _ = get_codebook(d, bits)
    ref_packed, ref_norms = encode(x, rotation, b, bits)
    ca = _UNPACK[bits](np.asarray(packed).reshape(-1, packed.shape[-1]), d)
    cb = _UNPACK[bits](ref_packed.reshape(-1, ref_packed.shape[-1]), d)
    x64 = np.asarray(x).reshape(-1, d).astype(np.float64)
    y64 = rotate_unit_f64(np.asarray(x).reshape(-1, d), rotation)
    with np.errstate(invalid="ignore", over="ignore"):
        unit64 = x64 / (np.linalg.norm(x64, axis=-1, keepdims=True) + 1e-10)
    n, max_ulps, hist = code_mismatch_report(ca, cb, y64, b, unit64, rotation)
    nr = np.asarray(ref_norms).reshape(-1).astype(np.float64)
    ng = np.asarray(norms).reshape(-1).astype(np.float64)
    nz = nr > 0
    rel = float(np.max(np.abs(ng[nz] - nr[nz]) / nr[nz])) if nz.any() else 0.0
    full = {"<=1": 0, "<=4": 0, "<=16": 0, ">16": 0}
    full.update({k: v for k, v in hist.items() if k in full})
    return {"codes": int(ca.size), "mismatching": int(n), "max_ulps_from_boundary": max_ulps,
            "ulp_histogram": full, "max_code_step": int(hist.get("max_code_step", 0)), "norm_max_rel_diff": rel}


def encode(x, rotation, boundaries, bits) -> Tuple[np.ndarray, np.ndarray]:
    """TurboQuant.encode, quantizer.py:122-166 (torch path :203-207)."""
    x = np.asarray(x)
    batch = x.shape[:-1]
    y, norms = rotate_unit(x, rotation)
    packed = _PACK[bits](quantize(y, boundaries, bits))
    return packed.reshape(batch + (packed.shape[-1],)), norms.reshape(batch)


def decode(packed, norms, rotation, centroids, bits, out_dtype=np.float16):
    """TurboQuant.decode, quantizer.py:168-197 (torch path :209-212)."""
    packed = np.asarray(packed, dtype=np.uint8)
    norms = np.asarray(norms)
    D = rotation.shape[0]
    batch = norms.shape
    idx = _UNPACK[bits](packed.reshape(-1, packed.shape[-1]), D)
    y_hat = np.asarray(centroids, dtype=f32)[idx.astype(np.int64)]
    x_hat = (y_hat @ rotation.astype(f32)) * norms.reshape(-1).astype(f32)[:, None]
    return x_hat.reshape(batch + (D,)).astype(out_dtype)


def batch_decompress_active_blocks(cache, norms, buf, block_table, num_blocks, rotation, centroids,
                                   bits, packed_dim):
    """One of the two (K, V) halves of TurboQuantImpl._batch_decompress_active_blocks,
    vllm/backend.py:1040-1091: unique ids of the block table inside [0, num_blocks) (:1061-1063),
    gather packed[:, :, :, :packed_dim] and norms (:1069-1075), one flat decode (:1083-1087),
    scatter into buf with a cast to its dtype (:1090-1091).  buf is written in place; blocks
    not listed keep their contents."""
    active = np.unique(np.asarray(block_table).reshape(-1))
    active = active[(active >= 0) & (active < num_blocks)]
    if active.size == 0:
        return
    A, (bs, H) = active.shape[0], cache.shape[1:3]
    flat_p = cache[active][:, :, :, :packed_dim].reshape(A * bs * H, packed_dim)
    flat_n = norms[active].reshape(A * bs * H)
    dec = decode(flat_p, flat_n, rotation, centroids, bits)       # float16, as tq.decode returns
    buf[active] = dec.reshape(A, bs, H, -1).astype(buf.dtype)


# --------------------------------------------------------------------------------------
# fused_kv_update.py (torch fallback = semantics of record)
# --------------------------------------------------------------------------------------
def kv_update(x, slot_mapping, out_packed, out_norms, rotation, boundaries, block_size=16,
              max_blocks=0, bits=4):
    """_pytorch_tq4_kv_update, fused_kv_update.py:220-293 (generalised over bits): negative
    slots and blocks >= max_blocks are skipped; writes out_packed[blk, pos], out_norms[blk,
    pos] in place."""
    if max_blocks == 0:
        max_blocks = out_packed.shape[0]
    slot_mapping = np.asarray(slot_mapping)
    x = np.asarray(x)
    valid = slot_mapping >= 0
    blk = slot_mapping // block_size
    valid &= blk < max_blocks
    if not valid.any():
        return
    xs = x[valid]
    N, H, D = xs.shape
    packed, norms = encode(xs.reshape(N * H, D), rotation, boundaries, bits)
    b = blk[valid]
    p = slot_mapping[valid] % block_size
    out_packed[b, p] = packed.reshape(N, H, -1)
    out_norms[b, p] = norms.reshape(N, H)


# --------------------------------------------------------------------------------------
# fused_attention.py
# --------------------------------------------------------------------------------------
def paged_attention_loop(query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens,
                         rotation, centroids, bits, block_size=16, scale=None):
    """TQPagedAttentionRef.forward, fused_attention.py:91-185, literally: per (seq, q-head) an
    online softmax over tokens in float32; ctx == 0 leaves zeros; output in query dtype.
    Pure Python loops: small cases only."""
    query = np.asarray(query)
    S, QH, D = query.shape
    KVH = k_packed.shape[2]
    gqa = QH // KVH
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    scale = f32(scale)
    c = np.asarray(centroids, dtype=f32)
    R = rotation.astype(f32)
    out = np.zeros_like(query)
    for s in range(S):
        ctx = int(context_lens[s])
        if ctx == 0:
            continue
        nblk = math.ceil(ctx / block_size)
        for qh in range(QH):
            h = qh // gqa
            q_rot = R @ query[s, qh].astype(f32)
            m = f32(-np.inf)
            l = f32(0)
            acc = np.zeros(D, dtype=f32)
            for bi in range(nblk):
                phys = int(block_tables[s, bi])
                n_valid = min(block_size, ctx - bi * block_size)
                for pos in range(n_valid):
                    k = c[_UNPACK[bits](k_packed[phys, pos, h][None], D)[0].astype(np.int64)]
                    score = f32(np.dot(q_rot[0::2], k[0::2]) + np.dot(q_rot[1::2], k[1::2]))
                    score = f32(score * f32(k_norms[phys, pos, h]) * scale)
                    m_new = max(m, score)
                    with np.errstate(invalid="ignore"):
                        alpha = f32(np.exp(f32(m - m_new)))
                    beta = f32(np.exp(f32(score - m_new)))
                    l = f32(alpha * l + beta)
                    v = c[_UNPACK[bits](v_packed[phys, pos, h][None], D)[0].astype(np.int64)]
                    acc = alpha * acc + f32(beta * f32(v_norms[phys, pos, h])) * v
                    m = m_new
            if l > 0:
                acc = acc / l
            out[s, qh] = (R.T @ acc).astype(query.dtype)
    return out


def gather_dequant(packed, norms, block_tables, context_lens, centroids, bits, D, block_size,
                   dtype=f32):
    """Rotated-domain dequantisation of every token a sequence addresses:
    yields per sequence an array [ctx, KVH, D] = centroids[idx] * norm (no inverse rotation)."""
    c = np.asarray(centroids, dtype=dtype)
    res = []
    for s in range(len(context_lens)):
        ctx = int(context_lens[s])
        nblk = -(-ctx // block_size)
        blocks = np.asarray(block_tables[s, :nblk], dtype=np.int64)
        pk = packed[blocks].reshape((nblk * block_size,) + packed.shape[2:])[:ctx]
        nm = norms[blocks].reshape((nblk * block_size,) + norms.shape[2:])[:ctx]
        idx = _UNPACK[bits](pk, D).astype(np.int64)
        res.append(c[idx] * nm[..., None].astype(dtype))
    return res


def paged_attention(query, k_packed, k_norms, v_packed, v_norms, block_tables, context_lens,
                    rotation, centroids, bits, block_size=16, scale=None, dtype=f32,
                    cast_output=True):
    """Vectorised form of the same computation (softmax over all tokens at once instead of the
    running max/sum of fused_attention.py:141-163 -- equal in exact arithmetic).  `dtype`
    float64 gives a higher-precision judge for tolerance checks."""
    query = np.asarray(query)
    S, QH, D = query.shape
    KVH = k_packed.shape[2]
    gqa = QH // KVH
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    R = rotation.astype(dtype)
    out = np.zeros((S, QH, D), dtype=dtype)
    kd = gather_dequant(k_packed, k_norms, block_tables, context_lens, centroids, bits, D,
                        block_size, dtype)
    vd = gather_dequant(v_packed, v_norms, block_tables, context_lens, centroids, bits, D,
                        block_size, dtype)
    for s in range(S):
        if int(context_lens[s]) == 0:
            continue
        q_rot = query[s].astype(dtype) @ R.T                       # [QH, D]
        q_rot = q_rot.reshape(KVH, gqa, D)
        sc = np.einsum("hgd,thd->hgt", q_rot, kd[s]) * dtype(scale)
        sc -= sc.max(axis=-1, keepdims=True)
        p = np.exp(sc)
        p /= p.sum(axis=-1, keepdims=True)
        acc = np.einsum("hgt,thd->hgd", p, vd[s]).reshape(QH, D)
        out[s] = acc @ R
    return out.astype(query.dtype) if cast_output else out


# --------------------------------------------------------------------------------------
# block_selector.py
# --------------------------------------------------------------------------------------
def block_rep_update(acc_even, acc_odd, counts, block_indices, k_packed, k_norms, centroids):
    """BlockRepresentativeCache.update, block_selector.py:66-101: per new token and kv head the
    norm-weighted centroids of the high / low nibbles are added to the block's accumulators and
    the block's count goes up by one.  In place."""
    kp = np.asarray(k_packed).astype(np.int64)
    c = np.asarray(centroids, dtype=f32)
    kn = np.asarray(k_norms, dtype=f32)[..., None]
    we = kn * c[(kp >> 4) & 0xF]
    wo = kn * c[kp & 0xF]
    bi = np.asarray(block_indices)
    np.add.at(acc_even, bi, we)
    np.add.at(acc_odd, bi, wo)
    np.add.at(counts, bi, 1)


def block_rep_finalize(acc_even, acc_odd, counts, rep_even, rep_odd, block_indices=None):
    """BlockRepresentativeCache.finalize, block_selector.py:103-118: rep = acc / max(count, 1)
    for the given blocks (all when None).  In place."""
    sel = slice(None) if block_indices is None else np.asarray(block_indices)
    safe = np.maximum(counts[sel], 1)[..., None].astype(f32)
    rep_even[sel] = acc_even[sel] / safe
    rep_odd[sel] = acc_odd[sel] / safe


def block_scores(q_even, q_odd, rep_even, rep_odd, block_tables, context_lens, gqa_ratio, block_size):
    """score_blocks, block_selector.py:129-179: mean query of each GQA group against the
    representatives of the table's blocks (ids clamped at 0), summed over kv heads and
    coordinates; columns at or beyond ceil(ctx / block_size) are -inf."""
    S, QH, HD = q_even.shape
    KV = QH // gqa_ratio
    qe = q_even.reshape(S, KV, gqa_ratio, HD).mean(axis=2, dtype=f32)
    qo = q_odd.reshape(S, KV, gqa_ratio, HD).mean(axis=2, dtype=f32)
    bt = np.maximum(np.asarray(block_tables), 0)
    ge, go = rep_even[bt], rep_odd[bt]                            # [S, B, KV, HD]
    sc = (qe[:, None] * ge).sum(axis=(-1, -2), dtype=f32) + (qo[:, None] * go).sum(axis=(-1, -2), dtype=f32)
    nb = (np.asarray(context_lens) + block_size - 1) // block_size
    sc = sc.astype(f32)
    sc[np.arange(bt.shape[1])[None, :] >= nb[:, None]] = -np.inf
    return sc


def block_select(scores, block_tables, context_lens, block_size, max_selected, num_sink_blocks=2,
                 num_recent_blocks=2):
    """select_blocks, block_selector.py:182-236: sink and recent columns forced in, top-k of the
    rest (k = min(max_selected, table width)), kept in column order, physical ids gathered,
    zero padding up to max_selected; context = min(ctx, k * block_size).  Among equal scores (the
    two zeros are equal) the lower column wins here (torch.topk leaves that open); a NaN score ranks
    above everything, +inf included, as torch.topk ranks it."""
    scores = np.asarray(scores, dtype=f32)
    S, B = scores.shape
    ctx = np.asarray(context_lens)
    nb = (ctx + block_size - 1) // block_size
    col = np.arange(B)[None, :]
    valid = col < nb[:, None]
    mandatory = ((col < num_sink_blocks) | (col >= nb[:, None] - num_recent_blocks)) & valid
    sel = scores.copy()
    sel[mandatory] = np.inf
    sel[~valid] = -np.inf
    k = min(max_selected, B)
    nan = np.isnan(sel)
    finite_key = np.where(nan, np.inf, sel)
    order = np.stack([np.lexsort((np.arange(B), -finite_key[s], ~nan[s])) for s in range(S)]) if S else np.zeros((0, B), int)
    top = np.sort(order[:, :k], axis=1)
    fbt = np.take_along_axis(np.asarray(block_tables), top, axis=1)
    if k < max_selected:
        fbt = np.concatenate([fbt, np.zeros((S, max_selected - k), dtype=fbt.dtype)], axis=1)
    fcl = np.minimum(ctx, k * block_size).astype(ctx.dtype)
    return fbt, fcl


# --------------------------------------------------------------------------------------
# hybrid_quantizer.py (tq35 and tq25, calibrate_uniform)
# --------------------------------------------------------------------------------------
def fwht(x):
    """fwht_pow2, hybrid_quantizer.py:130-151: unnormalised Walsh-Hadamard butterflies over the
    last axis (power of two)."""
    x = np.array(x, dtype=f32, copy=True)
    n = x.shape[-1]
    h = 1
    while h < n:
        v = x.reshape(x.shape[:-1] + (-1, 2 * h))
        a = v[..., :h].copy()
        b = v[..., h:].copy()
        v[..., :h] = a + b
        v[..., h:] = a - b
        h *= 2
    return x


def fwht_general(x):
    """fwht_general, hybrid_quantizer.py:154-193: a length that is no power of two is cut into
    descending powers of two (96 = 64 + 32) and every piece is transformed on its own."""
    x = np.asarray(x, dtype=f32)
    n = x.shape[-1]
    if n > 0 and (n & (n - 1)) == 0:
        return fwht(x)
    out, at = np.array(x, dtype=f32, copy=True), 0
    while n > 0:
        p = 1 << (n.bit_length() - 1)
        out[..., at:at + p] = fwht(x[..., at:at + p])
        at, n = at + p, n - p
    return out


def structured_hadamard(x, signs, inverse=False):
    """structured_hadamard, hybrid_quantizer.py:200-234 with normalized=True (the division by
    sqrt(dim) is a float32 division by the float32 value of the square root, as torch's CPU
    kernel divides a float32 tensor by a Python number)."""
    dim = x.shape[-1]
    if inverse:
        y = fwht_general(x) * signs
    else:
        y = fwht_general(x * signs)
    return (y / f32(math.sqrt(dim))).astype(f32)


def dimension_aware_codebook(dim: int, bits: int):
    """dimension_aware_codebook, hybrid_quantizer.py:241-303: 200-iteration Lloyd on a
    10,000-point grid weighted by (1-x^2)^((d-3)/2), float64, cast to float32."""
    L = 1 << bits
    n = 10000
    start, end = -0.999, 0.999
    step = (end - start) / (n - 1)
    i = np.arange(n, dtype=np.float64)
    # torch.linspace fills the upper half from the end point
    grid = np.where(i < n // 2, start + step * i, end - step * (n - 1 - i))
    w = (1.0 - grid * grid) ** ((dim - 3) / 2.0)
    w = w / w.sum()
    step_c = (grid[-1] - grid[0]) / (L - 1)
    j = np.arange(L, dtype=np.float64)
    c = np.where(j < L // 2, grid[0] + step_c * j, grid[-1] - step_c * (L - 1 - j))
    for _ in range(200):
        b = (c[:-1] + c[1:]) / 2.0
        a = np.clip(np.searchsorted(b, grid, side="left"), 0, L - 1)
        new = c.copy()
        for k in range(L):
            m = a == k
            ws = w[m].sum()
            if ws > 1e-30:
                new[k] = (grid[m] * w[m]).sum() / ws
        done = np.abs(c - new).max() < 1e-10
        c = new
        if done:
            break
    return c.astype(f32), ((c[:-1] + c[1:]) / 2.0).astype(f32)


def pack_multibit(idx, bits):
    """pack_multibit, hybrid_quantizer.py:310-352: MSB-first bit stream over the last axis."""
    idx = np.asarray(idx).astype(np.int64)
    dim = idx.shape[-1]
    flat = idx.reshape(-1, dim) & ((1 << bits) - 1)
    nbytes = math.ceil(dim * bits / 8)
    bitsarr = np.zeros((flat.shape[0], nbytes * 8), dtype=np.uint8)
    for b in range(bits):
        bitsarr[:, b:dim * bits:bits] = (flat >> (bits - 1 - b)) & 1
    return np.packbits(bitsarr, axis=-1, bitorder="big").reshape(idx.shape[:-1] + (nbytes,))


def unpack_multibit(packed, dim, bits):
    """unpack_multibit, hybrid_quantizer.py:355-396."""
    packed = np.asarray(packed, dtype=np.uint8)
    flat = packed.reshape(-1, packed.shape[-1])
    bitsarr = np.unpackbits(flat, axis=-1, bitorder="big")[:, :dim * bits]
    v = np.zeros((flat.shape[0], dim), dtype=np.uint8)
    for b in range(bits):
        v = (v << 1) | bitsarr[:, b::bits]
    return v.reshape(packed.shape[:-1] + (dim,))


class HybridParams:
    """The constants HybridTurboQuant(head_dim=128, mode) holds after calibrate_uniform():
    hybrid_quantizer.py:52-65,92-123,486-547,590-603.  tq35: dims 0..63 at 3 bits and 64..127 at
    2 bits (64-byte rows); tq25: dims 0..31 at 2 bits and 32..127 at 1 bit (44-byte rows).
    The sign vectors come from torch's CPU generator (seed 42) and are arguments."""

    def __init__(self, g0_had, g1_had, g0_qjl, g1_qjl, head_dim=128, codebooks=None, mode="tq35"):
        assert head_dim == 128
        self.head_dim = head_dim
        self.mode = mode
        self.g_dim = {"tq35": (64, 64), "tq25": (32, 96)}[mode]
        self.mse_bits = {"tq35": (3, 2), "tq25": (2, 1)}[mode]
        self.had = (np.asarray(g0_had, f32), np.asarray(g1_had, f32))
        self.qjl = (np.asarray(g0_qjl, f32), np.asarray(g1_qjl, f32))
        assert self.had[0].shape == (self.g_dim[0],) and self.had[1].shape == (self.g_dim[1],)
        if codebooks is None:
            codebooks = tuple(dimension_aware_codebook(self.g_dim[g], self.mse_bits[g]) for g in (0, 1))
        self.centroids = (codebooks[0][0], codebooks[1][0])
        self.boundaries = (codebooks[0][1], codebooks[1][1])
        self.qjl_scale = tuple(math.sqrt(math.pi / 2.0) / self.g_dim[g] for g in (0, 1))
        # byte layout: [mse | qjl bits | norm fp16 | residual norm fp16] per group
        self.mse_bytes = tuple(-(-self.g_dim[g] * self.mse_bits[g] // 8) for g in (0, 1))
        self.sign_bytes = tuple(-(-self.g_dim[g] // 8) for g in (0, 1))
        self.group_bytes = tuple(self.mse_bytes[g] + self.sign_bytes[g] + 4 for g in (0, 1))
        self.packed_dim = sum(self.group_bytes)


def _hybrid_encode_group(xg, hp: HybridParams, g):
    """_encode_single_group, hybrid_quantizer.py:706-779."""
    xg = xg.astype(f32)
    n = np.sqrt(np.sum(xg * xg, axis=-1, dtype=f32)).astype(f32)
    unit = xg / (n[:, None] + f32(1e-10))
    rot = structured_hadamard(unit, hp.had[g])
    idx = np.clip(np.searchsorted(hp.boundaries[g], rot, side="left"), 0, (1 << hp.mse_bits[g]) - 1)
    mse_packed = pack_multibit(idx, hp.mse_bits[g])
    mse_hat = structured_hadamard(hp.centroids[g][idx], hp.had[g], inverse=True)
    res = (unit - mse_hat).astype(f32)
    rn = np.sqrt(np.sum(res * res, axis=-1, dtype=f32)).astype(f32)
    proj = structured_hadamard(res, hp.qjl[g])
    qjl_packed = pack_multibit((proj >= 0).astype(np.uint8), 1)
    nb = n.astype(np.float16).view(np.uint8).reshape(-1, 2)
    rb = rn.astype(np.float16).view(np.uint8).reshape(-1, 2)
    return np.concatenate([mse_packed, qjl_packed, nb, rb], axis=-1)


def hybrid_encode(x, hp: HybridParams):
    """HybridTurboQuant.encode with calibrate_uniform groups (the first g0 dims / the rest),
    hybrid_quantizer.py:616-704."""
    x = np.asarray(x)
    flat = x.reshape(-1, 128).astype(f32)
    d0 = hp.g_dim[0]
    out = np.concatenate([_hybrid_encode_group(flat[:, :d0], hp, 0),
                          _hybrid_encode_group(flat[:, d0:], hp, 1)], axis=-1)
    return out.reshape(x.shape[:-1] + (hp.packed_dim,))


def _hadamard_matrix(n):
    """Float64 matrix of fwht_general over n points (block diagonal for 96 = 64 + 32), unnormalised."""
    out, at = np.zeros((n, n)), 0
    while n - at > 0:
        p = 1 << ((n - at).bit_length() - 1)
        h = np.array([[1.0]])
        while h.shape[0] < p:
            h = np.block([[h, h], [h, -h]])
        out[at:at + p, at:at + p] = h
        at += p
    return out


def hybrid_encode_margins(x, packed, hp: HybridParams):
    """Float64 account of every bit of `packed` (rows produced by ANY float32 implementation of
    hybrid_encode for the vectors `x`): how far the quantity behind each code, each sign bit and
    each stored norm lies from the value at which that bit would flip.  A float32 implementation
    may differ from another one (summation order of the norm and of the butterflies) only where
    these margins are a few float32 ulps; anywhere else a difference is a defect.

    For both groups g, with the codes and signs READ FROM `packed` (so that a code which
    legitimately flipped does not make the signs that follow from it look wrong):
      code_ulps[g]  [n,64]  |rot64 - boundary| for the farthest boundary the stored code would have
                            to cross to reach the float64 code, in float32 ulps of the larger of that
                            boundary and the row's largest |rot64| (0 where the codes agree)
      sign_ulps[g]  [n,64]  |proj64| in float32 ulps of the row's largest |proj64| where the stored
                            sign differs from sign(proj64), else 0
      norm_steps[g], rnorm_steps[g]  [n]  stored fp16 norm / residual norm minus the fp16 rounding
                            of the float64 value, in fp16 steps (bit patterns)
    Same operations as _hybrid_encode_group (hybrid_quantizer.py:706-779) carried in float64."""
    x = np.asarray(x).reshape(-1, 128).astype(f32).astype(np.float64)
    packed = np.asarray(packed, dtype=np.uint8).reshape(-1, hp.packed_dim)
    out = {"code_ulps": [], "sign_ulps": [], "norm_steps": [], "rnorm_steps": []}
    for g, (lo, off) in enumerate(((0, 0), (hp.g_dim[0], hp.group_bytes[0]))):
        G = hp.g_dim[g]
        # (the reference divides by the float32 value of sqrt(dim))
        H = _hadamard_matrix(G) / float(f32(math.sqrt(G)))
        xg = x[:, lo:lo + G]
        pg = packed[:, off:off + hp.group_bytes[g]]
        mb, sb = hp.mse_bytes[g], hp.sign_bytes[g]
        n64 = np.sqrt(np.sum(xg * xg, axis=-1))
        # the reference divides by the float32 norm + 1e-10 (float32 arithmetic)
        unit = xg / (n64.astype(f32) + f32(1e-10)).astype(np.float64)[:, None]
        had = hp.had[g].astype(np.float64)
        rot = (unit * had) @ H
        b = hp.boundaries[g].astype(np.float64)
        idx64 = np.clip(np.searchsorted(b, rot, side="left"), 0, (1 << hp.mse_bits[g]) - 1)
        idx = unpack_multibit(pg[:, :mb], G, hp.mse_bits[g]).astype(np.int64)
        # boundaries between the stored code and the float64 code: the farthest one decides
        far = np.where(idx > idx64, b[np.clip(idx - 1, 0, len(b) - 1)], b[np.clip(idx, 0, len(b) - 1)])
        # the rounding error of a butterfly sum is absolute, of the size of the terms summed: a result
        # that cancels to (nearly) zero is no more accurate than the row's large outputs
        floor = np.max(np.abs(rot), axis=-1, keepdims=True)
        ulp = np.spacing(np.maximum(np.maximum(np.maximum(np.abs(far), np.abs(rot)), floor), 1e-30).astype(f32)).astype(np.float64)
        out["code_ulps"].append(np.where(idx != idx64, np.abs(rot - far) / ulp, 0.0))
        mse_hat = (hp.centroids[g].astype(np.float64)[idx] @ H) * had
        res = unit - mse_hat
        rn64 = np.sqrt(np.sum(res * res, axis=-1))
        proj = (res * hp.qjl[g].astype(np.float64)) @ H
        sgn = unpack_multibit(pg[:, mb:mb + sb], G, 1).astype(bool)
        row_ulp = np.spacing(np.maximum(np.max(np.abs(proj), axis=-1), 1e-30).astype(f32)).astype(np.float64)
        out["sign_ulps"].append(np.where(sgn != (proj >= 0), np.abs(proj) / row_ulp[:, None], 0.0))
        for key, val, at in (("norm_steps", n64, mb + sb), ("rnorm_steps", rn64, mb + sb + 2)):
            stored = np.ascontiguousarray(pg[:, at:at + 2]).view(np.uint16).reshape(-1).astype(np.int64)
            want = val.astype(np.float16).view(np.uint16).astype(np.int64)
            out[key].append(stored - want)
    return out


def _hybrid_decode_group(pg, hp: HybridParams, g):
    """_decode_single_group, hybrid_quantizer.py:876-933."""
    mb, sb, G = hp.mse_bytes[g], hp.sign_bytes[g], hp.g_dim[g]
    idx = unpack_multibit(pg[:, :mb], G, hp.mse_bits[g]).astype(np.int64)
    mse_hat = structured_hadamard(hp.centroids[g][idx], hp.had[g], inverse=True)
    sgn = 2.0 * unpack_multibit(pg[:, mb:mb + sb], G, 1).astype(f32) - 1.0
    qjl_hat = structured_hadamard((sgn * f32(hp.qjl_scale[g])).astype(f32), hp.qjl[g], inverse=True)
    n = np.ascontiguousarray(pg[:, mb + sb:mb + sb + 2]).view(np.float16).reshape(-1).astype(f32)
    rn = np.ascontiguousarray(pg[:, mb + sb + 2:mb + sb + 4]).view(np.float16).reshape(-1).astype(f32)
    return ((mse_hat + qjl_hat * rn[:, None]) * n[:, None]).astype(f32)


def hybrid_decode(packed, hp: HybridParams):
    """HybridTurboQuant.decode, hybrid_quantizer.py:785-874; returns float32."""
    packed = np.asarray(packed, dtype=np.uint8)
    flat = packed.reshape(-1, hp.packed_dim)
    b0 = hp.group_bytes[0]
    out = np.concatenate([_hybrid_decode_group(flat[:, :b0], hp, 0),
                          _hybrid_decode_group(flat[:, b0:], hp, 1)], axis=-1)
    return out.reshape(packed.shape[:-1] + (128,))


def dense_attention(query, keys, values, scale, dtype=f32):
    """softmax(q K^T * scale) V for one sequence with GQA: query [QH,D], keys/values [T,KVH,D]."""
    QH, D = query.shape
    KVH = keys.shape[1]
    g = QH // KVH
    q = query.astype(dtype).reshape(KVH, g, D)
    sc = np.einsum("hgd,thd->hgt", q, keys.astype(dtype)) * dtype(scale)
    sc -= sc.max(axis=-1, keepdims=True)
    p = np.exp(sc)
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("hgt,thd->hgd", p, values.astype(dtype)).reshape(QH, D)


def hybrid_paged_attention(query, k_cache, v_cache, block_tables, context_lens, hp: HybridParams,
                           scale, block_size=16, dtype=f32):
    """tq::hybrid_decode_step's attention (vllm/hooks.py:294-345) in float32: decompress every
    addressed token with hybrid_decode, mask by context length, dense softmax attention.
    Caches are [blocks, block_size, KVH, hp.packed_dim] uint8.  Returns float32 [S, QH, D]."""
    query = np.asarray(query)
    S, QH, D = query.shape
    out = np.zeros((S, QH, D), dtype=dtype)
    for s in range(S):
        ctx = int(context_lens[s])
        if ctx == 0:
            continue
        nblk = -(-ctx // block_size)
        blocks = np.asarray(block_tables[s, :nblk], dtype=np.int64)
        kp = k_cache[blocks].reshape((-1,) + k_cache.shape[2:])[:ctx]
        vp = v_cache[blocks].reshape((-1,) + v_cache.shape[2:])[:ctx]
        out[s] = dense_attention(query[s], hybrid_decode(kp, hp), hybrid_decode(vp, hp), scale,
                                 dtype)
    return out


# --------------------------------------------------------------------------------------
# triattention/
# --------------------------------------------------------------------------------------
def rope_frequencies(head_dim, base=1_000_000.0):
    """spectral.py:34-51: theta_i = base ** (-2 i / d), evaluated in float32."""
    i = np.arange(head_dim // 2, dtype=f32)
    return np.power(f32(base), (f32(-2.0) * i) / f32(head_dim)).astype(f32)


def spectral_encode(x, num_freqs=12, coeff_bits=4):
    """SpectralKVEncoder.encode, encoder.py:73-149: top-F pairs by energy, indices ascending; then by width
      4   per-token max-abs scale (clamped at 1e-8), codes = clamp(round((v/scale + 1) * 7.5), 0, 15),
          byte = code_even << 4 | code_odd, scale -> fp16                                 (:118-133)
      8   the same with half-code 127.5 and range 0..255, the two codes of a pair in consecutive bytes:
          packed [..., 2F] uint8                                                          (:135-147)
      16  the pairs themselves rounded to fp16: packed [..., F, 2] float16, scales = 1    (:107-115)"""
    x = np.asarray(x)
    D = x.shape[-1]
    pairs = x.astype(f32).reshape(x.shape[:-1] + (D // 2, 2))
    en = np.sum(pairs * pairs, axis=-1, dtype=f32)
    order = np.argsort(-en, axis=-1, kind="stable")[..., :num_freqs]
    top = np.sort(order, axis=-1)
    tp = np.take_along_axis(pairs, top[..., None], axis=-2)
    if coeff_bits == 16:
        return top.astype(np.uint8), tp.astype(np.float16), np.ones(x.shape[:-1], dtype=np.float16)
    if coeff_bits not in (4, 8):
        raise ValueError(f"Unsupported coeff_bits: {coeff_bits}")
    half, top_code = (f32(7.5), 15) if coeff_bits == 4 else (f32(127.5), 255)
    scales = np.maximum(np.abs(tp).reshape(tp.shape[:-2] + (-1,)).max(axis=-1), f32(1e-8))
    nrm = tp / scales[..., None, None]
    q = np.clip(np.round((nrm + f32(1)) * half), 0, top_code).astype(np.uint8)
    if coeff_bits == 4:
        packed = ((q[..., 0] << 4) | q[..., 1]).astype(np.uint8)
    else:
        packed = q.reshape(q.shape[:-2] + (2 * num_freqs,))
    return top.astype(np.uint8), packed, scales.astype(np.float16)


def unpack_coefficients(packed, scales, coeff_bits=4):
    """TrigSeriesScorer._unpack_coefficients, scorer.py:84-113: (code / half - 1) * scale in float32 for
    4 bits (nibbles, half 7.5) and 8 bits (byte pairs, half 127.5); the fp16 pairs as they are for 16."""
    packed = np.asarray(packed)
    if coeff_bits == 16:
        return packed[..., 0].astype(f32), packed[..., 1].astype(f32)
    s = np.asarray(scales).astype(f32)[..., None]
    if coeff_bits == 4:
        v0, v1, half = (packed >> 4).astype(f32), (packed & 0x0F).astype(f32), f32(7.5)
    elif coeff_bits == 8:
        raw = packed.astype(f32).reshape(packed.shape[:-1] + (packed.shape[-1] // 2, 2))
        v0, v1, half = raw[..., 0], raw[..., 1], f32(127.5)
    else:
        raise ValueError(f"Unsupported coeff_bits: {coeff_bits}")
    return ((v0 / half - f32(1.0)) * s).astype(f32), ((v1 / half - f32(1.0)) * s).astype(f32)


def tri_scores(query, k_idx, k_packed, k_scales, theta, query_pos=None, key_positions=None, coeff_bits=4,
               pre_rope=True):
    """TrigSeriesScorer.score, scorer.py:115-208 -> [B, QH, S] float32 logits.  pre_rope: the trigonometric
    series over the position difference (:180-199); otherwise the plain sparse dot product sum_f c_f
    (:200-202), positions unused."""
    query = np.asarray(query)
    B, QH, D = query.shape
    S, KVH = k_idx.shape[1], k_idx.shape[2]
    gqa = QH // KVH
    if key_positions is None:
        key_positions = np.broadcast_to(np.arange(S)[None], (B, S))
    if query_pos is None:
        query_pos = np.full((B,), S)
    k0, k1 = unpack_coefficients(k_packed, k_scales, coeff_bits)  # [B,S,KVH,F]
    hmap = np.arange(QH) // gqa
    idx = k_idx.astype(np.int64)[:, :, hmap].transpose(0, 2, 1, 3)  # [B,QH,S,F]
    k0 = k0[:, :, hmap].transpose(0, 2, 1, 3)
    k1 = k1[:, :, hmap].transpose(0, 2, 1, 3)
    qf = query.astype(f32)
    qe = np.take_along_axis(np.broadcast_to(qf[..., 0::2][:, :, None], (B, QH, S, D // 2)), idx, -1)
    qo = np.take_along_axis(np.broadcast_to(qf[..., 1::2][:, :, None], (B, QH, S, D // 2)), idx, -1)
    c = qe * k0 + qo * k1
    if pre_rope:
        s = qo * k0 - qe * k1
        delta = (np.asarray(key_positions).astype(f32).reshape(B, 1, S, 1)
                 - np.asarray(query_pos).astype(f32).reshape(B, 1, 1, 1))
        ph = (delta * np.asarray(theta, dtype=f32)[idx]).astype(f32)
        raw = np.sum(c * np.cos(ph) + s * np.sin(ph), axis=-1, dtype=f32)
    else:
        raw = np.sum(c, axis=-1, dtype=f32)
    return (raw * f32(1.0 / math.sqrt(D))).astype(f32)


def tri_decode_step(query, k_enc, v_enc, theta, query_pos=None, key_positions=None, coeff_bits=4,
                    pre_rope=True, mask=None):
    """TriAttention.decode_step, attention.py:186-280: scores -> softmax over S -> weighted
    scatter-add of the value coefficients into even/odd bins -> interleave.  k_enc / v_enc are
    (indices, packed, scales) triples.  `mask` [B, 1, S] is added to the logits first, which makes
    this one query position of TriAttention.forward (attention.py:148-170).  Returns float32 [B, QH, D]."""
    query = np.asarray(query)
    B, QH, D = query.shape
    sc = tri_scores(query, *k_enc, theta, query_pos, key_positions, coeff_bits, pre_rope)
    if mask is not None:
        sc = (sc + np.asarray(mask, dtype=f32)).astype(f32)
    sc = sc - sc.max(axis=-1, keepdims=True)
    w = np.exp(sc)
    w = (w / w.sum(axis=-1, keepdims=True, dtype=f32)).astype(f32)
    v_idx, v_packed, v_scales = v_enc
    KVH = v_idx.shape[2]
    gqa = QH // KVH
    v0, v1 = unpack_coefficients(v_packed, v_scales, coeff_bits)   # [B,S,KVH,F]
    out = np.zeros((B, QH, D), dtype=f32)
    for b in range(B):
        for qh in range(QH):
            h = qh // gqa
            ii = v_idx[b, :, h].astype(np.int64).reshape(-1)
            wv0 = (w[b, qh][:, None] * v0[b, :, h]).reshape(-1)
            wv1 = (w[b, qh][:, None] * v1[b, :, h]).reshape(-1)
            np.add.at(out[b, qh], 2 * ii, wv0)
            np.add.at(out[b, qh], 2 * ii + 1, wv1)
    return out


def spectral_fetch_sequence(cache_arrays, block_table, context_len, block_size):
    """SpectralKVCache.fetch_sequence, triattention/cache.py:163-198: the first
    ceil(context_len / block_size) entries of the block table select physical blocks, whose tokens
    are laid end to end and cut at context_len.  cache_arrays: the six pool arrays
    (k_indices, k_packed, k_scales, v_indices, v_packed, v_scales), each [num_blocks, block_size, ...].
    Returns (k_enc, v_enc) triples with a leading axis of context_len."""
    nb = -(-int(context_len) // block_size)
    phys = np.asarray(block_table)[:nb].astype(np.int64)
    got = [np.asarray(a)[phys].reshape((-1,) + np.asarray(a).shape[2:])[:context_len] for a in cache_arrays]
    return tuple(got[:3]), tuple(got[3:])


def tri_decode_step_paged(query, cache_arrays, block_tables, context_lens, block_size, theta, query_pos=None,
                          coeff_bits=4, pre_rope=True):
    """A batch of sequences in one block pool: per sequence fetch_sequence then decode_step with the
    default key positions 0..ctx-1 and query position ctx (scorer.py:142-146); an empty sequence
    gives zeros (softmax over no tokens, nothing scattered).  Returns float32 [B, QH, D]."""
    query = np.asarray(query)
    B, QH, D = query.shape
    out = np.zeros((B, QH, D), dtype=f32)
    for b in range(B):
        n = int(context_lens[b])
        if n <= 0:
            continue
        k_enc, v_enc = spectral_fetch_sequence(cache_arrays, block_tables[b], n, block_size)
        qp = None if query_pos is None else np.asarray(query_pos)[b:b + 1]
        out[b] = tri_decode_step(query[b:b + 1], tuple(a[None] for a in k_enc), tuple(a[None] for a in v_enc),
                                 theta, qp, None, coeff_bits, pre_rope)[0]
    return out

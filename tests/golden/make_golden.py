#!/usr/bin/env python3
"""Write the golden vectors under tests/golden/ by running the reference on the CPU.

Run once, in the build container only (the reference tree is not available where
the GPU tests run):

    python tests/golden/make_golden.py [/root/reference]

The reference's own tests hold no golden vectors, and the following results are
fixed by nothing but the reference's code running on torch's CPU generator /
LAPACK, so they are captured here as data (inputs and expected outputs only):

  * random_orthogonal(128|64, seed=42)            rotation.py:20-35
  * dimension_aware_codebook(64, 3|2)             hybrid_quantizer.py:241-303
  * the four tq35 sign vectors                    hybrid_quantizer.py:514-523
  * rope_frequencies(128, 1e6), (32, 1e4)         triattention/spectral.py:34-51
  * TurboQuant.encode / decode, 2/3/4-bit         quantizer.py:122-212
  * _pytorch_tq4_kv_update scatter semantics      fused_kv_update.py:220-293
  * TQPagedAttentionRef.forward, 2/3/4-bit        fused_attention.py:91-185
  * HybridTurboQuant tq35 encode / decode         hybrid_quantizer.py:616-933
  * SpectralKVEncoder.encode, TriAttention.decode_step
                                                  triattention/encoder.py:73-149,
                                                  triattention/attention.py:186-280

Inputs come from numpy's PCG64 (`default_rng(seed)`), and are stored next to the
outputs so the tests never depend on a generator's bit stream.
"""
import math
import os
import sys

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, REF)
HERE = os.path.dirname(os.path.abspath(__file__))

from aither_kvcache.rotation import random_orthogonal  # noqa: E402
from aither_kvcache.quantizer import TurboQuant  # noqa: E402
from aither_kvcache.fused_kv_update import _pytorch_tq4_kv_update  # noqa: E402
from aither_kvcache.fused_attention import TQPagedAttentionRef  # noqa: E402
from aither_kvcache.hybrid_quantizer import (  # noqa: E402
    HybridTurboQuant, dimension_aware_codebook)
from aither_kvcache.triattention.config import TriAttentionConfig  # noqa: E402
from aither_kvcache.triattention.attention import TriAttention  # noqa: E402
from aither_kvcache.triattention.spectral import rope_frequencies  # noqa: E402

torch.set_num_threads(1)  # fixed summation order inside MKL for the record


def kv_like(rng, shape):
    """fp16 vectors: N(0,1) entries times a lognormal(0, 0.5) scale per vector."""
    g = rng.standard_normal(shape, dtype=np.float32)
    s = rng.lognormal(0.0, 0.5, size=shape[:-1]).astype(np.float32)
    return (g * s[..., None]).astype(np.float16)


out = {}

# ---- init-time constants -------------------------------------------------------------
for d in (64, 128):
    out[f"rotation_d{d}_seed42"] = random_orthogonal(d, seed=42, device="cpu").numpy()
out["rotation_d128_seed7"] = random_orthogonal(128, seed=7, device="cpu").numpy()
for bits in (3, 2):
    c, b = dimension_aware_codebook(64, bits)
    out[f"hyb_centroids_64_{bits}"] = c.numpy()
    out[f"hyb_boundaries_64_{bits}"] = b.numpy()
htq = HybridTurboQuant(head_dim=128, mode="tq35", seed=42, device="cpu")
out["hyb_g0_had_signs"] = htq._g0_had_signs.numpy()
out["hyb_g1_had_signs"] = htq._g1_had_signs.numpy()
out["hyb_g0_qjl_signs"] = htq._g0_qjl_signs.numpy()
out["hyb_g1_qjl_signs"] = htq._g1_qjl_signs.numpy()
out["theta_d128_base1e6"] = rope_frequencies(128, 1_000_000.0).numpy()
out["theta_d32_base1e4"] = rope_frequencies(32, 10000.0).numpy()

# ---- uniform TurboQuant encode / decode ----------------------------------------------
rng = np.random.default_rng(100)
x_enc = kv_like(rng, (96, 128))
x_enc[5] = 0  # zero vector: y == boundary[mid] == 0.0 tie, and norm 0
out["enc_x"] = x_enc
for bits in (2, 3, 4):
    tq = TurboQuant(head_dim=128, bits=bits, seed=42, device="cpu")
    out[f"centroids_b{bits}"] = tq.centroids.numpy()
    out[f"boundaries_b{bits}"] = tq.boundaries_inner.numpy()
    packed, norms = tq.encode(torch.from_numpy(x_enc))
    out[f"enc_packed_b{bits}"] = packed.numpy()
    out[f"enc_norms_b{bits}"] = norms.numpy()
    out[f"dec_b{bits}"] = tq.decode(packed, norms).numpy()  # fp16
# f32 and bf16 inputs, 4-bit
tq4 = TurboQuant(head_dim=128, bits=4, seed=42, device="cpu")
x32 = (rng.standard_normal((16, 128)) * 3.0).astype(np.float32)
out["enc_x_f32"] = x32
p, n = tq4.encode(torch.from_numpy(x32))
out["enc_packed_f32_b4"], out["enc_norms_f32_b4"] = p.numpy(), n.numpy()
xb = torch.from_numpy(x32).to(torch.bfloat16)
out["enc_x_bf16_as_f32"] = xb.float().numpy()
p, n = tq4.encode(xb)
out["enc_packed_bf16_b4"], out["enc_norms_bf16_b4"] = p.numpy(), n.numpy()
# head_dim 64 (another supported power of two)
tq64 = TurboQuant(head_dim=64, bits=4, seed=42, device="cpu")
x64 = kv_like(rng, (32, 64))
out["enc_x_d64"] = x64
p, n = tq64.encode(torch.from_numpy(x64))
out["enc_packed_d64_b4"], out["enc_norms_d64_b4"] = p.numpy(), n.numpy()
out["dec_d64_b4"] = tq64.decode(p, n).numpy()

# ---- paged scatter semantics ---------------------------------------------------------
rng = np.random.default_rng(101)
T, H, NB, BS = 24, 2, 6, 16
xk = kv_like(rng, (T, H, 128))
slots = rng.permutation(NB * BS)[:T].astype(np.int64)
slots[3] = -1            # padding token
slots[7] = NB * BS + 5   # block index beyond the cache
slots[11] = 4 * BS + 2   # block 4 while max_blocks=4 is passed below -> skipped
kp = torch.zeros(NB, BS, H, 64, dtype=torch.uint8)
kn = torch.zeros(NB, BS, H)
_pytorch_tq4_kv_update(torch.from_numpy(xk), torch.from_numpy(slots), kp, kn,
                       tq4.rotation, tq4.boundaries_inner, BS, NB)
out["upd_x"], out["upd_slots"] = xk, slots
out["upd_packed"], out["upd_norms"] = kp.numpy(), kn.numpy()
kp2 = torch.zeros(NB, BS, H, 64, dtype=torch.uint8)
kn2 = torch.zeros(NB, BS, H)
_pytorch_tq4_kv_update(torch.from_numpy(xk), torch.from_numpy(slots), kp2, kn2,
                       tq4.rotation, tq4.boundaries_inner, BS, 4)
out["upd_packed_max4"], out["upd_norms_max4"] = kp2.numpy(), kn2.numpy()

# ---- paged decode attention (the reference's torch loop) -----------------------------
rng = np.random.default_rng(102)
S, QH, KVH, BS, NB = 4, 8, 2, 16, 12
ctx = np.array([0, 21, 48, 37], dtype=np.int64)
tables = np.full((S, 3), 0, dtype=np.int64)
perm = rng.permutation(NB)
tables[1, :2] = perm[0:2]
tables[2, :3] = perm[2:5]
tables[3, :3] = perm[5:8]
tables[1, 2] = 10**6     # padding beyond ceil(ctx/bs): must never be dereferenced
keys = kv_like(rng, (NB * BS, KVH, 128))
vals = kv_like(rng, (NB * BS, KVH, 128))
q = rng.standard_normal((S, QH, 128), dtype=np.float32).astype(np.float16)
out["attn_q"], out["attn_keys"], out["attn_vals"] = q, keys, vals
out["attn_tables"], out["attn_ctx"] = tables, ctx
for bits in (2, 3, 4):
    tq = TurboQuant(head_dim=128, bits=bits, seed=42, device="cpu")
    kp, kn = tq.encode(torch.from_numpy(keys))
    vp, vn = tq.encode(torch.from_numpy(vals))
    P = kp.shape[-1]
    kp, vp = kp.reshape(NB, BS, KVH, P), vp.reshape(NB, BS, KVH, P)
    kn, vn = kn.reshape(NB, BS, KVH), vn.reshape(NB, BS, KVH)
    ref = TQPagedAttentionRef(tq.rotation, tq.centroids, 1.0 / math.sqrt(128), KVH, QH, 128,
                              BS, bits=bits)
    o = ref.forward(torch.from_numpy(q), kp, kn, vp, vn, torch.from_numpy(tables),
                    torch.from_numpy(ctx))
    out[f"attn_kp_b{bits}"], out[f"attn_kn_b{bits}"] = kp.numpy(), kn.numpy()
    out[f"attn_vp_b{bits}"], out[f"attn_vn_b{bits}"] = vp.numpy(), vn.numpy()
    out[f"attn_out_b{bits}"] = o.numpy()  # fp16, query dtype

# ---- hybrid tq35 ---------------------------------------------------------------------
rng = np.random.default_rng(103)
xh = kv_like(rng, (40, 128))
xh[9] = 0
htq.calibrate_uniform(num_kv_heads=1)
ph = htq.encode(torch.from_numpy(xh))
out["hyb_x"], out["hyb_packed"] = xh, ph.numpy()
out["hyb_decoded"] = htq.decode(ph).numpy()  # f32
htq8 = HybridTurboQuant(head_dim=128, mode="tq35", seed=42, device="cpu")
htq8.calibrate_uniform(num_kv_heads=2)
xh2 = kv_like(rng, (6, 2, 128))
ph2 = htq8.encode(torch.from_numpy(xh2))
out["hyb_x_heads2"], out["hyb_packed_heads2"] = xh2, ph2.numpy()
out["hyb_decoded_heads2"] = htq8.decode(ph2).numpy()

# ---- TriAttention --------------------------------------------------------------------
rng = np.random.default_rng(104)
cfg = TriAttentionConfig(head_dim=128, num_freqs=12, coeff_bits=4, num_kv_heads=2,
                         num_query_heads=8, rope_base=1_000_000.0)
tri = TriAttention(cfg, device="cpu")
B, S = 2, 80
pair_std = (np.arange(64) + 1.0) ** -0.75
tk = (rng.standard_normal((B, S, 2, 64, 2)) * pair_std[:, None]).reshape(B, S, 2, 128)
tk = tk.astype(np.float16)
tv = rng.standard_normal((B, S, 2, 128)).astype(np.float16)
tq_ = rng.standard_normal((B, 8, 128)).astype(np.float32)
k_enc, v_enc = tri.encode_kv(torch.from_numpy(tk), torch.from_numpy(tv))
out["tri_keys"], out["tri_vals"], out["tri_q"] = tk, tv, tq_
for nm, e in (("k", k_enc), ("v", v_enc)):
    out[f"tri_{nm}_indices"] = e.indices.numpy()
    out[f"tri_{nm}_packed"] = e.packed.numpy()
    out[f"tri_{nm}_scales"] = e.scales.numpy()
out["tri_out_default_pos"] = tri.decode_step(torch.from_numpy(tq_), k_enc, v_enc).numpy()
qpos = np.array([30000, 517], dtype=np.int64)
kpos = np.stack([np.arange(S) * 3 + 11, np.arange(S)[::-1] * 7]).astype(np.int64)
out["tri_qpos"], out["tri_kpos"] = qpos, kpos
out["tri_out_explicit_pos"] = tri.decode_step(
    torch.from_numpy(tq_), k_enc, v_enc, torch.from_numpy(qpos), torch.from_numpy(kpos)).numpy()
out["tri_scores_explicit_pos"] = tri.scorer.score(
    torch.from_numpy(tq_), k_enc, torch.from_numpy(qpos), torch.from_numpy(kpos)).numpy()

np.savez_compressed(os.path.join(HERE, "golden_v1.npz"), **out)
total = sum(v.nbytes for v in out.values())
print(f"wrote {len(out)} arrays, {total/1024:.1f} KiB raw ->",
      os.path.getsize(os.path.join(HERE, "golden_v1.npz")) // 1024, "KiB on disk")

#!/usr/bin/env python3
"""Write tests/golden/golden_tri_widths.npz by running the reference's TriAttention on the CPU with the
coefficient widths and the scoring mode its default configuration does not use.

Run once, in the build container only (the reference tree is not available where the GPU tests run):

    python tests/golden/make_golden_tri_widths.py [/root/reference]

The reference's tests hold no vectors for these, so the results of

  * SpectralKVEncoder.encode, coeff_bits 8 and 16        triattention/encoder.py:73-149
  * TrigSeriesScorer.score, coeff_bits 8 and 16,         triattention/scorer.py:74-113,115-208
    and pre_rope=False (post-RoPE: plain sparse dot product) at 4 / 8 / 16 bits
  * TriAttention.decode_step with those                   triattention/attention.py:186-280

are captured here as data (inputs and expected outputs only).  Inputs come from numpy's PCG64.
"""
import os
import sys

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, REF)
HERE = os.path.dirname(os.path.abspath(__file__))

from aither_kvcache.triattention.config import TriAttentionConfig  # noqa: E402
from aither_kvcache.triattention.attention import TriAttention  # noqa: E402

torch.set_num_threads(1)
rng = np.random.default_rng(21)
out = {}

B, S, KVH, QH, D, F = 2, 45, 2, 8, 128, 12
pair_std = (np.arange(D // 2) + 1.0) ** -0.75
keys = (rng.standard_normal((B, S, KVH, D // 2, 2)) * pair_std[:, None]).reshape(B, S, KVH, D).astype(np.float16)
vals = rng.standard_normal((B, S, KVH, D)).astype(np.float16)
q = rng.standard_normal((B, QH, D)).astype(np.float32)
qpos = np.array([S + 3, 4000], dtype=np.int64)
kpos = np.sort(rng.integers(0, 3000, size=(B, S)), axis=-1).astype(np.int64)
out["keys"], out["vals"], out["q"], out["qpos"], out["kpos"] = keys, vals, q, qpos, kpos

for bits in (4, 8, 16):
    for pre in (True, False):
        if bits == 4 and pre:
            continue                     # the default configuration: covered by the main golden file
        cfg = TriAttentionConfig(head_dim=D, num_freqs=F, coeff_bits=bits, num_kv_heads=KVH, num_query_heads=QH,
                                 rope_base=1e6, pre_rope=pre)
        tri = TriAttention(cfg, device="cpu")
        k_enc, v_enc = tri.encode_kv(torch.from_numpy(keys), torch.from_numpy(vals))
        tag = f"b{bits}_{'pre' if pre else 'post'}"
        if pre or bits == 4:             # encodings do not depend on the scoring mode: stored once per width
            for nm, e in (("k", k_enc), ("v", v_enc)):
                out[f"enc_b{bits}_{nm}_indices"] = e.indices.numpy()
                out[f"enc_b{bits}_{nm}_packed"] = e.packed.numpy()
                out[f"enc_b{bits}_{nm}_scales"] = e.scales.numpy()
        out[f"scores_{tag}"] = tri.scorer.score(torch.from_numpy(q), k_enc, torch.from_numpy(qpos),
                                                torch.from_numpy(kpos)).numpy()
        out[f"out_{tag}"] = tri.decode_step(torch.from_numpy(q), k_enc, v_enc, torch.from_numpy(qpos),
                                            torch.from_numpy(kpos)).numpy()
        out[f"out_default_pos_{tag}"] = tri.decode_step(torch.from_numpy(q), k_enc, v_enc).numpy()

path = os.path.join(HERE, "golden_tri_widths.npz")
np.savez_compressed(path, **out)
print("wrote", path, {k: v.shape for k, v in out.items()})

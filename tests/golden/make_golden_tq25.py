#!/usr/bin/env python3
"""Write tests/golden/golden_tq25.npz by running the reference's HybridTurboQuant in mode tq25 on the CPU.

Run once, in the build container only (the reference tree is not available where the GPU tests run):

    python tests/golden/make_golden_tq25.py [/root/reference]

The reference's tests hold no vectors for this mode and nothing else fixes its bits (the sign vectors
come from torch's generator, the one-bit codebook's only boundary is what the grid iteration's float64
summation leaves near zero), so the results of

  * the four sign vectors of seed 42                      hybrid_quantizer.py:514-523
  * dimension_aware_codebook(32, 2) and (96, 1)           hybrid_quantizer.py:241-303
  * HybridTurboQuant(mode="tq25").encode / decode         hybrid_quantizer.py:616-933
    (groups of 32 and 96 coordinates, the 96-point transform as a 64- and a 32-point block,
    hybrid_quantizer.py:154-193)

are captured here as data (inputs and expected outputs only).  Inputs come from numpy's PCG64.
"""
import os
import sys

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, REF)
HERE = os.path.dirname(os.path.abspath(__file__))

from aither_kvcache.hybrid_quantizer import HybridTurboQuant, dimension_aware_codebook  # noqa: E402

torch.set_num_threads(1)
out = {}

htq = HybridTurboQuant(head_dim=128, mode="tq25", seed=42, device="cpu")
out["g0_had"], out["g1_had"] = htq._g0_had_signs.numpy(), htq._g1_had_signs.numpy()
out["g0_qjl"], out["g1_qjl"] = htq._g0_qjl_signs.numpy(), htq._g1_qjl_signs.numpy()
for nm, (dim, bits) in (("g0", (32, 2)), ("g1", (96, 1))):
    c, b = dimension_aware_codebook(dim, bits)
    out[f"{nm}_centroids"], out[f"{nm}_boundaries"] = c.numpy(), b.numpy()
out["packed_dim"] = np.array(htq.packed_dim, dtype=np.int64)

rng = np.random.default_rng(125)
# rows of different scales with a few large channels, as keys and values have them; one zero row, one row
# whose first group is zero
x = rng.standard_normal((48, 128)) * np.exp(rng.uniform(-3.0, 3.0, size=(48, 1)))
x[:, rng.integers(0, 128, size=5)] *= 6.0
x[7] = 0
x[11, :32] = 0
x = x.astype(np.float32)
htq.calibrate_uniform(num_kv_heads=1)
p = htq.encode(torch.from_numpy(x))
out["x"], out["packed"] = x, p.numpy()
out["decoded"] = htq.decode(p).numpy()

htq2 = HybridTurboQuant(head_dim=128, mode="tq25", seed=42, device="cpu")
htq2.calibrate_uniform(num_kv_heads=2)
x2 = rng.standard_normal((5, 2, 128)).astype(np.float16)
p2 = htq2.encode(torch.from_numpy(x2))
out["x_heads2"], out["packed_heads2"] = x2, p2.numpy()
out["decoded_heads2"] = htq2.decode(p2).numpy()

np.savez_compressed(os.path.join(HERE, "golden_tq25.npz"), **out)
print("wrote golden_tq25.npz:", {k: v.shape for k, v in out.items()})

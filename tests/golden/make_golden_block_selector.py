#!/usr/bin/env python3
"""Write tests/golden/golden_block_selector.npz by running the reference's block selector on the CPU.

Run once, in the build container only (the reference tree is not available where the GPU tests run):

    python tests/golden/make_golden_block_selector.py [/root/reference]

The reference's tests hold no vectors for block_selector.py, so the results of

  * BlockRepresentativeCache.update / finalize      block_selector.py:66-118
  * score_blocks                                    block_selector.py:129-179
  * select_blocks                                   block_selector.py:182-236
  * BlockSelector.update_reps / select              block_selector.py:282-337

are captured here as data (inputs and expected outputs only).  Inputs come from numpy's PCG64.
Scores are continuous random numbers, so no two candidates of a top-k tie; the mandatory (sink /
recent) blocks never exceed the number selected.
"""
import os
import sys

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, REF)
HERE = os.path.dirname(os.path.abspath(__file__))

from aither_kvcache.block_selector import (  # noqa: E402
    BlockRepresentativeCache, BlockSelector, score_blocks, select_blocks)
from aither_kvcache.codebook import get_codebook  # noqa: E402

torch.set_num_threads(1)
rng = np.random.default_rng(11)
out = {}

centroids = get_codebook(128, 4)[0]
centroids = torch.as_tensor(np.asarray(centroids), dtype=torch.float32)
out["centroids"] = centroids.numpy()

# ---- representatives: 3 update calls over 12 blocks, 2 kv heads, packed_dim 64
MB, H, PD = 12, 2, 64
cache = BlockRepresentativeCache(MB, H, PD, torch.device("cpu"), centroids)
for call, n in enumerate((40, 1, 23)):
    bi = rng.integers(0, MB - 2, size=n).astype(np.int64)          # blocks 10, 11 stay empty
    pos = rng.integers(0, 16, size=n).astype(np.int64)
    kp = rng.integers(0, 256, size=(n, H, PD), dtype=np.uint8)
    kn = rng.lognormal(2.0, 0.5, size=(n, H)).astype(np.float32)
    cache.update(torch.from_numpy(bi), torch.from_numpy(pos), torch.from_numpy(kp), torch.from_numpy(kn))
    cache.finalize(torch.from_numpy(np.unique(bi)))
    out[f"rep_bi_{call}"], out[f"rep_pos_{call}"], out[f"rep_kp_{call}"], out[f"rep_kn_{call}"] = bi, pos, kp, kn
    out[f"rep_even_after_{call}"] = cache.rep_even.numpy().copy()
    out[f"rep_odd_after_{call}"] = cache.rep_odd.numpy().copy()
    out[f"rep_counts_after_{call}"] = cache._counts.numpy().copy()
cache.clear_blocks(torch.tensor([3, 4]))
cache.finalize()
out["rep_even_cleared"] = cache.rep_even.numpy().copy()
out["rep_counts_cleared"] = cache._counts.numpy().copy()

# ---- scores and selection: 3 sequences, 8 query / 2 kv heads, 100 table columns, 300 physical blocks
S, QH, KVH, HD, BPS, NB, BS = 3, 8, 2, 64, 100, 300, 16
q_even = rng.standard_normal((S, QH, HD)).astype(np.float32)
q_odd = rng.standard_normal((S, QH, HD)).astype(np.float32)
rep_even = rng.standard_normal((NB, KVH, HD)).astype(np.float32)
rep_odd = rng.standard_normal((NB, KVH, HD)).astype(np.float32)
ctx = np.array([100 * BS - 5, 37 * BS, 3 * BS + 1], dtype=np.int64)      # 100, 37 and 4 blocks
bt = np.full((S, BPS), -1, dtype=np.int64)
for s in range(S):
    nb = (ctx[s] + BS - 1) // BS
    bt[s, :nb] = rng.permutation(NB)[:nb]
scores = score_blocks(torch.from_numpy(q_even), torch.from_numpy(q_odd), torch.from_numpy(rep_even),
                      torch.from_numpy(rep_odd), torch.from_numpy(bt), torch.from_numpy(ctx), QH // KVH, BS)
for k, v in (("q_even", q_even), ("q_odd", q_odd), ("rep_even", rep_even), ("rep_odd", rep_odd), ("ctx", ctx), ("bt", bt)):
    out["sel_" + k] = v
out["sel_scores"] = scores.numpy()
for max_sel in (10, 40, 120):
    fbt, fcl = select_blocks(scores, torch.from_numpy(bt), torch.from_numpy(ctx), BS, max_sel, 2, 2)
    out[f"sel_fbt_{max_sel}"], out[f"sel_fcl_{max_sel}"] = fbt.numpy(), fcl.numpy()
fbt, fcl = select_blocks(scores, torch.from_numpy(bt), torch.from_numpy(ctx), BS, 12, 1, 3)
out["sel_fbt_12_s1r3"], out["sel_fcl_12_s1r3"] = fbt.numpy(), fcl.numpy()

# ---- the orchestrating class: ratio 0.1 of 300 blocks -> 30 selected
sel = BlockSelector(NB, KVH, HD, torch.device("cpu"), centroids, select_ratio=0.1, min_blocks_for_selection=64)
sel._rep_cache.rep_even.copy_(torch.from_numpy(rep_even))
sel._rep_cache.rep_odd.copy_(torch.from_numpy(rep_odd))
fbt, fcl = sel.select(torch.from_numpy(q_even), torch.from_numpy(q_odd), torch.from_numpy(bt), torch.from_numpy(ctx), QH // KVH, BS)
out["cls_max_selected"] = np.array(sel.max_selected)
out["cls_fbt"], out["cls_fcl"] = fbt.numpy(), fcl.numpy()

np.savez_compressed(os.path.join(HERE, "golden_block_selector.npz"), **out)
print(f"wrote {len(out)} arrays,", os.path.getsize(os.path.join(HERE, "golden_block_selector.npz")) // 1024, "KiB on disk")

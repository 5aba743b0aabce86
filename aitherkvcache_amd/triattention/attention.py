"""TriAttention decode step on MI355X (reference: aither_kvcache/triattention/attention.py:186-280
with TrigSeriesScorer.score, scorer.py:115-208).

score(q, k_t) = (1/sqrt d) sum_f [ c_f cos(delta theta_f) + s_f sin(delta theta_f) ] over the
token's retained RoPE pairs (config.pre_rope; otherwise the keys were stored after RoPE and the score is
(1/sqrt d) sum_f c_f, scorer.py:200-202), coefficients of 4, 8 or 16 bits (scorer.py:84-113), softmax over the cached tokens, and a weighted scatter-add of the
value coefficients -- one HIP kernel over the spectral cache plus a merge kernel, instead of the
reference's chain of [B, QH, S, F] float32 temporaries.
"""
import math
from typing import Optional, Tuple

import torch

from .. import _lib
from .config import TriAttentionConfig
from .encoder import SpectralEncoding, SpectralKVEncoder, packed_shape, unpack_coefficients
from .scorer import TrigSeriesScorer
from .spectral import rope_frequencies


class TriAttention:
    def __init__(self, config: TriAttentionConfig, device: str = "cpu"):
        self.config = config
        self.device = device
        self.head_dim = config.head_dim
        self.num_query_heads = config.num_query_heads
        self.num_kv_heads = config.num_kv_heads
        self.gqa_ratio = config.gqa_ratio
        self.scale = 1.0 / math.sqrt(config.head_dim)
        self.encoder = SpectralKVEncoder(config)
        self.scorer = TrigSeriesScorer(config, device=device)
        # float32 table evaluated on the host exactly as the reference does, then moved
        self._theta = rope_frequencies(config.head_dim, config.rope_base, device="cpu").to(device)
        self._workspace: Optional[torch.Tensor] = None

    def to(self, device: str) -> "TriAttention":
        self.device = device
        self._theta = self._theta.to(device)
        self.scorer.to(device)
        return self

    def encode_kv(self, keys: torch.Tensor, values: torch.Tensor) -> Tuple[SpectralEncoding, SpectralEncoding]:
        """keys / values [B, S, num_kv_heads, head_dim] (keys before RoPE)."""
        return self.encoder.encode(keys), self.encoder.encode(values)

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                positions: Optional[torch.Tensor] = None,
                attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Encode K / V, then attend every query position (reference: attention.py:116-182; its prefill form).
        query [B, QH, S_q, D] or [B, QH, D]; key / value [B, S_kv, KVH, D] (keys before RoPE); positions [B, S_kv]
        key positions (default 0..S_kv-1); query i sits at position i; attention_mask [B, S_q, S_kv] or
        [B, 1, S_kv], added to the logits (-inf = masked) -> float32 [B, QH, S_q, D] (or [B, QH, D]).
        Without a mask a query position is one decode_step; with one, the logits come from the scorer, mask and
        softmax are torch ops and the weighted sum of the sparse value rows is a scatter-add."""
        squeeze = query.dim() == 3
        if squeeze:
            query = query.unsqueeze(2)
        B, QH, S_q, D = query.shape
        k_enc, v_enc = self.encode_kv(key, value)
        outs = []
        for qi in range(S_q):
            q_i = query[:, :, qi, :]
            q_pos = torch.full((B,), qi, device=query.device, dtype=torch.int64)
            if attention_mask is None:
                outs.append(self.decode_step(q_i, k_enc, v_enc, q_pos, positions))
                continue
            scores = self.scorer.score(q_i, k_enc, q_pos, positions)
            mask_i = attention_mask[:, qi:qi + 1, :] if attention_mask.dim() == 3 and attention_mask.shape[1] > 1 \
                else attention_mask
            weights = torch.softmax(scores + mask_i.to(scores.dtype), dim=-1)
            outs.append(self._accumulate_values(weights, v_enc))
        out = torch.stack(outs, dim=2)
        return out.squeeze(2) if squeeze else out

    def _accumulate_values(self, weights: torch.Tensor, v_enc: SpectralEncoding) -> torch.Tensor:
        """sum_t weights[b, qh, t] * value row t of the query head's kv head, as float32 [B, QH, D]
        (reference: attention.py:219-280)."""
        B, QH, S = weights.shape
        KVH = v_enc.indices.shape[2]
        v0, v1 = unpack_coefficients(v_enc.packed, v_enc.scales, self.config.coeff_bits)       # [B, S, KVH, F]
        heads = torch.arange(QH, device=weights.device) // (QH // KVH)
        idx = v_enc.indices.long()[:, :, heads].permute(0, 2, 1, 3).reshape(B, QH, -1)           # [B, QH, S F]
        w = weights.unsqueeze(-1)
        out = torch.zeros(B, QH, self.head_dim, dtype=torch.float32, device=weights.device)
        out.scatter_add_(-1, idx * 2, (w * v0[:, :, heads].permute(0, 2, 1, 3)).reshape(B, QH, -1))
        out.scatter_add_(-1, idx * 2 + 1, (w * v1[:, :, heads].permute(0, 2, 1, 3)).reshape(B, QH, -1))
        return out

    @staticmethod
    def reference_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                            rope_base: float = 1_000_000.0, positions_q: Optional[torch.Tensor] = None,
                            positions_k: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Dense attention with explicit RoPE on the uncompressed tensors, for comparisons (reference:
        attention.py:285-345): query [B, QH, D] and key [B, S, KVH, D] before RoPE, value [B, S, KVH, D];
        positions default to S for the query and 0..S-1 for the keys -> float32 [B, QH, D].  Torch ops on the
        tensors' device."""
        B, QH, D = query.shape
        S, KVH = key.shape[1], key.shape[2]
        dev = query.device
        if positions_q is None:
            positions_q = torch.full((B,), S, device=dev)
        if positions_k is None:
            positions_k = torch.arange(S, device=dev).unsqueeze(0).expand(B, -1)
        theta = rope_frequencies(D, rope_base, device="cpu").to(dev)

        def rope(x, pos):                 # x [..., D], pos broadcastable to x.shape[:-1]
            ang = pos.float().unsqueeze(-1) * theta
            c, s = torch.cos(ang), torch.sin(ang)
            xe, xo = x.float()[..., 0::2], x.float()[..., 1::2]
            return torch.stack((xe * c - xo * s, xe * s + xo * c), dim=-1).flatten(-2)

        q = rope(query, positions_q.view(B, 1))                                   # [B, QH, D]
        k = rope(key, positions_k.view(B, S, 1))                                  # [B, S, KVH, D]
        heads = torch.arange(QH, device=dev) // (QH // KVH)
        scores = torch.einsum("bhd,bshd->bhs", q, k[:, :, heads]) / math.sqrt(D)
        w = torch.softmax(scores, dim=-1)
        return torch.einsum("bhs,bshd->bhd", w, value.float()[:, :, heads])

    def benchmark(self, batch_size: int = 1, seq_len: int = 2048, num_trials: int = 10) -> dict:
        """Times encode_kv, decode_step and the dense reference_attention on random data of the configured shape
        and compares the two results (reference: attention.py:347-405).  Wall-clock per call in milliseconds, the
        device synchronised around every timed loop."""
        import time
        dev = torch.device(self.device)
        D, QH, KVH = self.head_dim, self.num_query_heads, self.num_kv_heads
        q = torch.randn(batch_size, QH, D, device=dev)
        k = torch.randn(batch_size, seq_len, KVH, D, device=dev)
        v = torch.randn(batch_size, seq_len, KVH, D, device=dev)
        kpos = torch.arange(seq_len, device=dev).unsqueeze(0).expand(batch_size, -1).contiguous()
        qpos = torch.full((batch_size,), seq_len, device=dev)

        def timed(fn):
            res = fn()
            torch.cuda.synchronize(dev)
            t0 = time.perf_counter()
            for _ in range(num_trials):
                res = fn()
            torch.cuda.synchronize(dev)
            return res, (time.perf_counter() - t0) / num_trials * 1e3

        (k_enc, v_enc), enc_ms = timed(lambda: self.encode_kv(k, v))
        out, dec_ms = timed(lambda: self.decode_step(q, k_enc, v_enc, qpos, kpos))
        ref, ref_ms = timed(lambda: self.reference_attention(q, k, v, self.config.rope_base))
        cos = torch.nn.functional.cosine_similarity(out.reshape(-1, D).float(), ref.reshape(-1, D).float(), dim=-1)
        return {"encode_ms": enc_ms, "decode_ms": dec_ms, "reference_ms": ref_ms,
                "speedup": ref_ms / dec_ms if dec_ms > 0 else float("inf"),
                "compression_ratio": self.config.kv_compression_ratio,
                "cosine_similarity": cos.mean().item(), "mse": (out.float() - ref.float()).square().mean().item(),
                "seq_len": seq_len, "batch_size": batch_size}

    def decode_step(self, query: torch.Tensor, k_enc: SpectralEncoding, v_enc: SpectralEncoding,
                    query_pos: Optional[torch.Tensor] = None,
                    key_positions: Optional[torch.Tensor] = None) -> torch.Tensor:
        """query [B, QH, D]; encodings with indices/packed [B, S, KVH, F], scales [B, S, KVH];
        query_pos [B] (default S), key_positions [B, S] (default 0..S-1) -> float32 [B, QH, D]."""
        dev = _lib.require_gpu(query, k_enc.indices, k_enc.packed, k_enc.scales,
                               v_enc.indices, v_enc.packed, v_enc.scales, query_pos, key_positions)
        if self._theta.device != dev:
            self._theta = self._theta.to(dev)
        B, QH, D = query.shape
        _, S, KVH, F = k_enc.indices.shape
        if v_enc.indices.shape != k_enc.indices.shape:
            raise ValueError("k_enc and v_enc must have the same [B, S, KVH, F] shape")
        if D != self.head_dim or QH % KVH != 0:
            raise ValueError(f"bad shapes: query {tuple(query.shape)}, encodings {tuple(k_enc.indices.shape)}")
        q = query if query.dtype in (torch.float16, torch.bfloat16, torch.float32) else query.float()
        q = q.contiguous()

        cbits = self.config.coeff_bits
        cshape, cdtype = packed_shape([B, S, KVH], F, cbits)

        def u8(t):
            if t.dtype != torch.uint8:
                raise ValueError("indices must be uint8")
            return t.contiguous()

        def coeffs(t):
            if t.dtype != cdtype or list(t.shape) != cshape:
                raise ValueError(f"packed coefficients must be {cdtype} {cshape} at coeff_bits={cbits}, "
                                 f"got {t.dtype} {list(t.shape)}")
            return t.contiguous()

        ki, kc, vi, vc = u8(k_enc.indices), coeffs(k_enc.packed), u8(v_enc.indices), coeffs(v_enc.packed)
        ks = k_enc.scales.to(torch.float16).contiguous()
        vs = v_enc.scales.to(torch.float16).contiguous()

        def pos(t, shape):
            if t is None:
                return None
            if t.dtype not in (torch.int32, torch.int64):
                t = t.long()
            return t.expand(shape).contiguous()

        qp = pos(query_pos, (B,))
        kp = pos(key_positions, (B, S))
        out = torch.empty(B, QH, D, dtype=torch.float32, device=dev)
        L = _lib.lib()
        need = L.akv_tri_decode_workspace_bytes(B, QH, D)
        if self._workspace is None or self._workspace.numel() < need or self._workspace.device != dev:
            self._workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
        _lib.check(L.akv_tri_decode_step(
            q.data_ptr(), _lib.dtype_code(q), ki.data_ptr(), kc.data_ptr(), ks.data_ptr(),
            vi.data_ptr(), vc.data_ptr(), vs.data_ptr(), self._theta.data_ptr(),
            _lib.ptr(qp), _lib.itype_code(qp) if qp is not None else 0,
            _lib.ptr(kp), _lib.itype_code(kp) if kp is not None else 0,
            out.data_ptr(), B, S, QH, KVH, D, F, cbits, 1 if self.config.pre_rope else 0,
            self._workspace.data_ptr(), self._workspace.numel(), _lib.stream_ptr(dev)))
        return out

    def decode_step_paged(self, query: torch.Tensor, cache, block_tables: torch.Tensor,
                          context_lens: torch.Tensor, query_pos: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One decode step for a batch of sequences held in a SpectralKVCache: sequence b reads its
        first context_lens[b] tokens through block_tables[b] (what the reference does per sequence
        with cache.fetch_sequence, cache.py:163-198, followed by decode_step).  query [B, QH, D];
        block_tables [B, max_blocks_per_seq] int32/int64; context_lens [B]; key positions are
        0..ctx-1 and query_pos defaults to ctx -> float32 [B, QH, D] (zeros where ctx == 0)."""
        dev = _lib.require_gpu(query, cache.k_indices, cache.k_packed, cache.k_scales, cache.v_indices,
                               cache.v_packed, cache.v_scales, block_tables, context_lens, query_pos)
        if self._theta.device != dev:
            self._theta = self._theta.to(dev)
        B, QH, D = query.shape
        NB, BS, KVH, F = cache.k_indices.shape
        if D != self.head_dim or QH % KVH != 0:
            raise ValueError(f"query shape {tuple(query.shape)} does not fit head_dim={self.head_dim}, kv_heads={KVH}")
        if block_tables.dim() != 2 or block_tables.shape[0] != B or context_lens.numel() != B:
            raise ValueError("block_tables must be [B, max_blocks_per_seq] and context_lens [B]")
        q = query if query.dtype in (torch.float16, torch.bfloat16, torch.float32) else query.float()
        q = q.contiguous()
        for t in (cache.k_indices, cache.k_packed, cache.k_scales, cache.v_indices, cache.v_packed, cache.v_scales):
            if not t.is_contiguous():
                raise ValueError("the cache tensors must be contiguous")
        bt = block_tables if block_tables.dtype in (torch.int32, torch.int64) else block_tables.long()
        if bt.stride(1) != 1:
            bt = bt.contiguous()
        cl = context_lens if context_lens.dtype in (torch.int32, torch.int64) else context_lens.long()
        cl = cl.contiguous()
        qp = None
        if query_pos is not None:
            qp = query_pos if query_pos.dtype in (torch.int32, torch.int64) else query_pos.long()
            qp = qp.expand((B,)).contiguous()
        out = torch.empty(B, QH, D, dtype=torch.float32, device=dev)
        L = _lib.lib()
        need = L.akv_tri_decode_workspace_bytes(B, QH, D)
        if self._workspace is None or self._workspace.numel() < need or self._workspace.device != dev:
            self._workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
        rc = L.akv_tri_decode_paged(
            q.data_ptr(), _lib.dtype_code(q), cache.k_indices.data_ptr(), cache.k_packed.data_ptr(),
            cache.k_scales.data_ptr(), cache.v_indices.data_ptr(), cache.v_packed.data_ptr(),
            cache.v_scales.data_ptr(), self._theta.data_ptr(),
            _lib.ptr(qp), _lib.itype_code(qp) if qp is not None else 0,
            bt.data_ptr(), _lib.itype_code(bt), bt.stride(0), cl.data_ptr(), _lib.itype_code(cl),
            out.data_ptr(), B, NB, BS, bt.shape[1], QH, KVH, D, F, 1 if self.config.pre_rope else 0,
            self._workspace.data_ptr(), self._workspace.numel(), _lib.stream_ptr(dev))
        if rc == _lib.AKV_ERR_UNSUPPORTED:
            # shapes the paged kernel does not take: gather each sequence and use the dense-layout kernels
            lens = cl.tolist()
            for b in range(B):
                if lens[b] <= 0:
                    out[b].zero_()
                    continue
                k_enc, v_enc = cache.fetch_sequence(bt[b], lens[b])
                add = lambda e: SpectralEncoding(*(t.unsqueeze(0) for t in e))
                out[b] = self.decode_step(q[b:b + 1], add(k_enc), add(v_enc),
                                          None if qp is None else qp[b:b + 1])[0]
            return out
        _lib.check(rc)
        return out

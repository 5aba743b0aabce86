#!/usr/bin/env python3
"""Benchmark of the TurboQuant hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode4|decode4_b256|decode3|decode2|tq35|tq25|tri|encode]

A step is one pass of the hot path over one batch of synthetic input that is already resident
in HBM.  The default workload is the headline one: paged decode attention over a tq-t4nc cache
at the Llama-3-8B layer shape (32 query / 8 KV heads, head_dim 128, batch 16, context lengths
uniform in [1k, 40k], block_size 16, random non-contiguous block tables, seed 2), the cache
having been written by the encode-on-write kernel.  One JSON line is printed:

  value      algorithmic GB/s of the whole step (prologue + main + reduce kernels).  Before the W warm-up
             steps the step is called for 0.5 s (`config.preconditioning_s`), so that the K timed steps
             run at the device's sustained clocks like a serving loop, not as a cold burst
  roofline   the dominant kernel alone: algorithmic bytes / its mean duration, measured with HIP
             events on the launch stream (akv_profile_enable), against the 8 TB/s HBM peak
  cpu_baseline  the numpy oracle of the same computation timed on this box's host cores on a
             bounded sample of the same batch
  encode     the encode-on-write kernel: Mvec/s on 2**20 vectors, the latency of one 256-token
             step (K and V, 8 heads), and `sweep`: kernel duration for 2**12 .. 2**22 vectors with the
             smallest size that reaches 60 % of the HBM peak (`vectors_at_60pct_hbm`)
  hbm_reference  what a kernel that only reads (the library's read probe), torch's sum and a copy stream on this box over
             360 MB, the size of the headline step's cache: context for the fraction of the nominal peak

Algorithmic bytes per context token = 8 heads x (64 B codes + 4 B norm) x (K and V) = 1088 B
(104 / 72 / 128 / 88 B x 8 for 3-bit / 2-bit / tq35 / tq25), plus queries, outputs and block tables.
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def measured_traffic(workload):
    """HBM bytes per launch of the dominant kernel, from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE
    summary (counters scaled by a copy kernel of known size); None when no such run is on record."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f).get(workload)
    except OSError:
        return None
    return None if rec is None else rec["fetch_bytes"] + rec["write_bytes"]


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="decode4",
                    choices=["decode4", "decode4_b256", "decode3", "decode2", "tq35", "tq25", "tri", "encode"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the 3-bit / 2-bit / tq35 / tq25 / TriAttention workloads that the default run reports beside the headline one")
    ap.add_argument("--no-sweep", action="store_true",
                    help="skip the encode size sweep (a profiler run then sees the encode kernel at 2**20 vectors only)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 1 GiB device-to-device copy (a dispatch of known traffic, to scale "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    return ap.parse_args()


def lognormal_kv(torch, shape, gen, dev):
    """fp16 vectors: N(0,1) entries times a lognormal(0, 0.5) scale per vector."""
    g = torch.randn(shape, device=dev, generator=gen)
    s = torch.exp(0.5 * torch.randn(shape[:-1], device=dev, generator=gen))
    return (g * s.unsqueeze(-1)).half()


def profile_ms(L):
    ms = ctypes.c_float()
    rc = L.akv_profile_last_ms(ctypes.byref(ms))
    if rc != 0:
        raise RuntimeError(L.akv_last_error().decode())
    return ms.value


PRECONDITION_S = 0.5


def precondition(torch, fn, seconds=PRECONDITION_S):
    """Call the step for `seconds` so that the device sits at its sustained clocks, as in a serving loop
    that decodes continuously: a burst of a few milliseconds after an idle period runs 5-15 % slower on
    this part (same kernel, 95-99 us instead of 84-85 us) and says nothing about the kernel."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def timed(torch, fn, steps, warmup):
    precondition(torch, fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def kernel_ms(torch, L, fn, steps):
    """Mean duration of the dominant kernel over `steps` back-to-back calls (HIP events on the launch
    stream).  The library records one event pair per call into a ring of 64 and nothing is read back
    until the loop has ended, so the sampled calls run exactly like those of the timed region."""
    steps = max(1, min(int(steps), 64))
    precondition(torch, fn, PRECONDITION_S / 2)
    ms, n = ctypes.c_float(), ctypes.c_int()
    # the first sampled batch of a process reads 5-10 % high (the events of the ring are created and first
    # used there): one batch is sampled and dropped
    for _ in range(2):
        L.akv_profile_enable(1)
        for _ in range(steps):
            fn()
        rc = L.akv_profile_mean_ms(ctypes.byref(ms), ctypes.byref(n))
        L.akv_profile_enable(0)
        if rc != 0:
            break
    if rc != 0:
        raise RuntimeError(L.akv_last_error().decode())
    assert n.value == steps, (n.value, steps)
    return ms.value


def hbm_reference(torch, dev, L):
    """What plain streaming kernels reach on this box for a buffer of the workload's size (360 MB, two buffers
    alternated), in TB/s: the library's read probe (16-byte loads, nothing else; kernel time like the dominant
    kernels'), torch's sum (read only) and a device-to-device copy (read + write)."""
    n = 90 * 1024 * 1024
    xs = [torch.empty(n, dtype=torch.float32, device=dev).normal_() for _ in range(2)]
    y = torch.empty_like(xs[0])
    st = {"i": 0}

    def rd():
        st["i"] += 1
        xs[st["i"] & 1].sum()

    def cp():
        st["i"] += 1
        y.copy_(xs[st["i"] & 1])
    from aitherkvcache_amd import _lib
    sink = torch.zeros(64, dtype=torch.int32, device=dev)

    def probe():
        st["i"] += 1
        x = xs[st["i"] & 1]
        _lib.check(L.akv_debug_read_probe(x.data_ptr(), n * 4, sink.data_ptr(), _lib.stream_ptr(dev)))
    precondition(torch, rd, PRECONDITION_S / 2)
    t_rd = timed(torch, rd, 20, 5)
    t_cp = timed(torch, cp, 20, 5)
    t_pr = kernel_ms(torch, L, probe, 32)
    return {"bytes": n * 4, "read_probe_kernel_tbs": n * 4 / t_pr / 1e9, "torch_sum_read_tbs": n * 4 / t_rd / 1e9,
            "device_copy_read_plus_write_tbs": 2 * n * 4 / t_cp / 1e9}


# ---------------------------------------------------------------------------------------------
def bench_encode(torch, akv, L, dev, steps, warmup, cpu, cpu_seconds, sweep=True):
    tq = akv.TurboQuant(head_dim=128, bits=4, device=str(dev))
    gen = torch.Generator(device=dev).manual_seed(1)
    res = {}
    # (a) one serving step: 256 tokens x 8 heads, K and V, random free slots
    NB, BS, H, T = 8192, 16, 8, 256
    kp = torch.zeros(NB, BS, H, 64, dtype=torch.uint8, device=dev)
    vp = torch.zeros_like(kp)
    kn = torch.zeros(NB, BS, H, device=dev)
    vn = torch.zeros_like(kn)
    perm = torch.randperm(NB * BS, device=dev, generator=gen)
    k = lognormal_kv(torch, (T, H, 128), gen, dev)
    v = lognormal_kv(torch, (T, H, 128), gen, dev)
    slots = perm[:T].contiguous()

    class Cache:
        pass
    c = Cache()
    c.tq, c.block_size, c.max_blocks = tq, BS, NB
    c.k_packed, c.v_packed, c.k_norms, c.v_norms = kp[None], vp[None], kn[None], vn[None]
    step_ms = timed(torch, lambda: akv.fused_encode_and_store(c, 0, k, v, slots), steps, warmup)
    res["step_256tok_us"] = step_ms * 1e3
    res["step_256tok_bytes"] = 2 * T * H * 324 + T * 8
    # the kernel of that step by itself (events on its dispatch): what a caller without Python's call cost pays
    res["step_256tok_kernel_us"] = kernel_ms(torch, L, lambda: akv.fused_encode_and_store(c, 0, k, v, slots), 64) * 1e3
    # (b) bandwidth regime
    n = 1 << 20
    # two inputs alternated (2 x 268 MB): one alone would partly sit in the 256 MB last-level cache
    xs = [lognormal_kv(torch, (n, 128), gen, dev) for _ in range(2)]
    x = xs[0]
    st = {"i": 0}

    def enc_step():
        tq.encode(xs[st["i"] & 1])
        st["i"] += 1
    ms = timed(torch, enc_step, max(20, steps), 4)
    kms = kernel_ms(torch, L, enc_step, 32)
    res["vectors"] = n
    res["mvec_s"] = n / ms / 1e3
    res["kernel_mvec_s"] = n / kms / 1e3
    res["kernel_gbs"] = n * 324 / kms / 1e6
    res["kernel_frac_hbm"] = res["kernel_gbs"] / HBM_PEAK_GBS
    # the same vectors as float32 input (512 B read + 68 B written per vector)
    x32 = [v.float() for v in xs]

    def enc32_step():
        tq.encode(x32[st["i"] & 1])
        st["i"] += 1
    enc32_step()
    kms32 = kernel_ms(torch, L, enc32_step, 32)
    res["f32_input_kernel_mvec_s"] = n / kms32 / 1e3
    res["f32_input_kernel_gbs"] = n * 580 / kms32 / 1e6
    res["f32_input_kernel_frac_hbm"] = res["f32_input_kernel_gbs"] / HBM_PEAK_GBS
    del x32
    # decode of the same vectors (68 B in, 256 B out per vector)
    coded = [tq.encode(v) for v in xs]

    def dec_step():
        pk, nr = coded[st["i"] & 1]
        tq.decode(pk, nr)
        st["i"] += 1
    dms = timed(torch, dec_step, max(20, steps), 4)
    res["decode_mvec_s"] = n / dms / 1e3
    res["decode_gbs"] = n * 324 / dms / 1e6
    del coded, xs
    if sweep:
        res["sweep"], res["vectors_at_60pct_hbm"] = encode_sweep(torch, akv, L, tq, dev, gen)
    if cpu:
        from oracle import tq_oracle as O
        R = tq.rotation.cpu().numpy()
        _, b, _ = O.get_codebook(128, 4)
        xc = x[:65536].cpu().numpy()
        O.encode(xc[:4096], R, b, 4)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < cpu_seconds / 3 or reps < 2:
            O.encode(xc, R, b, 4)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_mvec_s"] = 65536 / dt / 1e6
        res["parity_config0"] = encode_parity_config0(torch, tq, dev, R)
    return res, tq


def encode_parity_config0(torch, tq, dev, R):
    """The 65,536 vectors of the CPU round-trip configuration (numpy PCG64 seed 0: N(0,1) entries times a
    lognormal(0, 0.5) norm, fp16) through the HIP encode and decode kernels, against the oracle: codes that
    differ, counted, with the distance of their float64 rotated value from the decision boundary in float32
    ulps as a histogram; norms; reconstruction error of the round trip."""
    from oracle import tq_oracle as O
    rng = np.random.default_rng(0)
    g = rng.standard_normal((65536, 128), dtype=np.float32)
    sc = rng.lognormal(0.0, 0.5, size=65536).astype(np.float32)
    x = (g * sc[:, None]).astype(np.float16)
    xd = torch.from_numpy(x).to(dev)
    packed, norms = tq.encode(xd)
    rep = O.encode_parity_report(packed.cpu().numpy(), norms.cpu().numpy(), x, R, 4)
    xh = tq.decode(packed, norms).float().cpu().numpy().astype(np.float64)
    x64 = x.astype(np.float64)
    rep["round_trip_mse"] = float(np.mean((xh - x64) ** 2))
    rep["round_trip_mse_over_mean_sq_norm"] = float(np.sum((xh - x64) ** 2) / np.sum(x64 ** 2))
    c, _, _ = O.get_codebook(128, 4)
    ref = O.decode(packed.cpu().numpy(), norms.cpu().numpy(), R, c, 4).astype(np.float64)
    rep["decode_max_abs_diff_vs_oracle"] = float(np.max(np.abs(xh - ref)))
    rep["vectors"] = 65536
    return rep


def decode_workload(torch, akv, dev, tq, bits_or_mode, seed, num_seqs, ctx):
    """Cache written through the HIP encode kernels + tables + queries."""
    gen = torch.Generator(device=dev).manual_seed(seed)
    rng = np.random.default_rng(seed)
    KVH, QH, BS = 8, 32, 16
    nblk = -(-ctx // BS)
    NB = int(nblk.sum())
    hybrid = bits_or_mode in ("tq35", "tq25")
    P = tq.layout.packed_dim if hybrid else tq._packed_dim
    kp = torch.zeros(NB, BS, KVH, P, dtype=torch.uint8, device=dev)
    vp = torch.zeros_like(kp)
    kn = vn = None
    if not hybrid:
        kn = torch.zeros(NB, BS, KVH, device=dev)
        vn = torch.zeros_like(kn)
    CH = 4096
    for b0 in range(0, NB, CH):
        b1 = min(NB, b0 + CH)
        slots = torch.arange(b0 * BS, b1 * BS, device=dev)
        for packed, norms in ((kp, kn), (vp, vn)):
            x = lognormal_kv(torch, ((b1 - b0) * BS, KVH, 128), gen, dev)
            if hybrid:
                akv.hybrid_encode_and_store(tq, x, slots, packed, BS)
            else:
                akv.fused_kv_update(x, slots, packed, norms, tq.rotation, tq.boundaries_inner, tq.bits, BS)
    perm = rng.permutation(NB)
    tables = np.zeros((num_seqs, int(nblk.max())), dtype=np.int32)
    off = 0
    for s in range(num_seqs):
        tables[s, :nblk[s]] = perm[off:off + nblk[s]]
        off += nblk[s]
    q = torch.randn(num_seqs, QH, 128, device=dev, generator=gen).half()
    return dict(kp=kp, kn=kn, vp=vp, vn=vn, tables_np=tables, ctx_np=ctx,
                tables=torch.from_numpy(tables).to(dev), ctx=torch.from_numpy(ctx.astype(np.int32)).to(dev),
                q=q, QH=QH, KVH=KVH, BS=BS, NB=NB)


def cpu_attention_baseline(w, tq, bits, seconds):
    """The oracle's vectorised float32 attention on whole sequences of the batch, shortest first,
    until the time budget is used."""
    from oracle import tq_oracle as O
    R = tq.rotation.cpu().numpy()
    c = tq.centroids.cpu().numpy()
    order = np.argsort(w["ctx_np"])
    q = w["q"].cpu().numpy()
    tokens = 0
    used = []
    t0 = time.perf_counter()
    for s in order:
        nb = -(-int(w["ctx_np"][s]) // 16)
        blocks = w["tables"][s, :nb].long()
        kp = w["kp"][blocks].cpu().numpy()
        kn = w["kn"][blocks].cpu().numpy()
        vp = w["vp"][blocks].cpu().numpy()
        vn = w["vn"][blocks].cpu().numpy()
        t1 = time.perf_counter()
        O.paged_attention(q[s:s + 1], kp, kn, vp, vn, np.arange(nb)[None], w["ctx_np"][s:s + 1], R, c, bits)
        dt = time.perf_counter() - t1
        tokens += int(w["ctx_np"][s])
        used.append((int(s), dt))
        if time.perf_counter() - t0 > seconds:
            break
    compute = sum(d for _, d in used)
    return tokens, compute, [s for s, _ in used]


def cpu_attention_loop_form(w, tq, bits, tokens=2048):
    """The reference's literal CPU attention (a Python loop per token, TQPagedAttentionRef.forward) on a slice:
    the longest sequence's first `tokens` tokens, one kv head and its four query heads.  Seconds per (token, kv head)."""
    from oracle import tq_oracle as O
    R = tq.rotation.cpu().numpy()
    c = tq.centroids.cpu().numpy()
    s = int(np.argmax(w["ctx_np"]))
    n = int(min(tokens, w["ctx_np"][s]))
    nb = -(-n // 16)
    blocks = w["tables"][s, :nb].long()
    kp, kn = w["kp"][blocks][:, :, :1].cpu().numpy(), w["kn"][blocks][:, :, :1].cpu().numpy()
    vp, vn = w["vp"][blocks][:, :, :1].cpu().numpy(), w["vn"][blocks][:, :, :1].cpu().numpy()
    q = w["q"][s:s + 1, :4].cpu().numpy()
    t0 = time.perf_counter()
    O.paged_attention_loop(q, kp, kn, vp, vn, np.arange(nb)[None], np.array([n]), R, c, bits)
    return (time.perf_counter() - t0) / n, n


def cpu_hybrid_baseline(w, tq, seconds):
    """The oracle's tq35 / tq25 attention (decompress every addressed row, dense softmax attention) on whole
    sequences of the batch, in batch order, until the time budget is used."""
    from oracle import tq_oracle as O
    tab = tq.kernel_table.cpu().numpy()
    if tq.mode == "tq25":
        hp = O.HybridParams(tab[0:32], tab[32:128], tab[128:160], tab[160:256],
                            codebooks=((tab[256:260], tab[262:265]), (tab[260:262], tab[265:266])), mode="tq25")
    else:
        hp = O.HybridParams(tab[0:64], tab[64:128], tab[128:192], tab[192:256],
                            codebooks=((tab[256:264], tab[268:275]), (tab[264:268], tab[275:278])))
    q = w["q"].float().cpu().numpy()
    tokens, compute, used = 0, 0.0, []
    t0 = time.perf_counter()
    for s in range(len(w["ctx_np"])):
        nb = -(-int(w["ctx_np"][s]) // 16)
        blocks = w["tables"][s, :nb].long()
        kc = w["kp"][blocks].cpu().numpy()
        vc = w["vp"][blocks].cpu().numpy()
        t1 = time.perf_counter()
        O.hybrid_paged_attention(q[s:s + 1], kc, vc, np.arange(nb)[None], w["ctx_np"][s:s + 1], hp,
                                 1 / math.sqrt(128))
        compute += time.perf_counter() - t1
        tokens += int(w["ctx_np"][s])
        used.append(s)
        if time.perf_counter() - t0 > seconds:
            break
    return tokens, compute, f"whole sequences {used} of the batch"


def encode_sweep(torch, akv, L, tq, dev, gen):
    """Encode kernel duration against problem size: T*H vectors of 128 fp16 for T*H = 2**12 .. 2**22
    (324 algorithmic bytes per vector).  Returns the rows and the smallest size at which the kernel
    reaches 60 % of the HBM peak (None if no size does)."""
    rows, reached = [], None
    for e in range(12, 23):
        n = 1 << e
        copies = max(2, min(8, (600 << 20) // (n * 256)))     # alternate inputs: more than the last-level cache
        xs = [lognormal_kv(torch, (n, 128), gen, dev) for _ in range(copies)]
        st = {"i": 0}

        def step():
            tq.encode(xs[st["i"] % copies])
            st["i"] += 1
        kms = kernel_ms(torch, L, step, 32)
        frac = n * 324 / kms / 1e6 / HBM_PEAK_GBS
        rows.append({"vectors": n, "kernel_us": round(kms * 1e3, 2), "frac_hbm": round(frac, 4)})
        if reached is None and frac >= 0.60:
            reached = n
        del xs
    return rows, reached


DECODE_DTYPE = "fp16 hi+lo MFMA operands (keys and queries carry 22 bits, values 11), f32 accumulate and softmax"


def traffic_fields(workload):
    """`traffic` of a roofline object: not measured in this run (counters need a profiler), read from the
    committed counter runs."""
    t = measured_traffic(workload)
    return {"traffic": t, "traffic_source": None if t is None else "profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / "
                                                                    "WRITE_SIZE runs of this command, committed; not measured in this run)"}


def run_decode(torch, akv, L, dev, workload, tq4, steps, warmup, cpu, cpu_seconds, cores):
    """One paged decode-attention workload: (result fields, roofline, cpu_baseline or None)."""
    if workload == "decode4":
        rng = np.random.default_rng(2)
        ctx = rng.integers(1024, 40961, size=16).astype(np.int64)
        name = "config 2: paged decode attention, tq-t4nc, 32Q/8KV d=128, batch 16, ctx U[1k,40k], block 16, seed 2"
        bits, per_tok, tq = 4, 1088, tq4
    elif workload == "decode4_b256":
        # a serving batch of many short sequences: the prologue and reduce kernels weigh as much as the main one
        ctx = np.full(256, 256, dtype=np.int64)
        name = "paged decode attention, tq-t4nc, 32Q/8KV d=128, batch 256 x 256 tokens, block 16, seed 2"
        bits, per_tok, tq = 4, 1088, tq4
    else:
        ctx = np.full(64, 8192, dtype=np.int64)
        bits = {"decode3": 3, "decode2": 2, "tq35": "tq35", "tq25": "tq25"}[workload]
        per_tok = {"decode3": 8 * 104, "decode2": 8 * 72, "tq35": 8 * 128, "tq25": 8 * 88}[workload]
        name = f"config 3: paged decode attention, {workload}, 32Q/8KV d=128, batch 64 x 8192, block 16, seed 3"
        if workload == "tq25":
            name = "paged decode attention, tq25 (a mode of the reference that none of its benchmark configurations uses; the shape of config 3), 32Q/8KV d=128, batch 64 x 8192, block 16, seed 3"
        if bits in ("tq35", "tq25"):
            tq = akv.HybridTurboQuant(mode=bits, device=str(dev))
            tq.calibrate_uniform(8)
        else:
            tq = akv.TurboQuant(head_dim=128, bits=bits, device=str(dev))
    seed = 2 if workload in ("decode4", "decode4_b256") else 3
    # two copies of the cache, alternated, so that no step finds its data in the 256 MB
    # last-level cache left by the previous one
    ws = [decode_workload(torch, akv, dev, tq, bits, seed + 100 * i, len(ctx), ctx) for i in range(2)]
    if bits in ("tq35", "tq25"):
        attn = akv.HybridPagedAttention(tq, 32)
        calls = [lambda w=w: attn.forward(w["q"], w["kp"], w["vp"], w["tables"], w["ctx"], scale=1 / math.sqrt(128))
                 for w in ws]
    else:
        attn = akv.TQPagedAttention(tq, 32)
        calls = [lambda w=w: attn.forward(w["q"], w["kp"], w["kn"], w["vp"], w["vn"], w["tables"], w["ctx"])
                 for w in ws]
    state = {"i": 0}

    def step():
        calls[state["i"] & 1]()
        state["i"] += 1

    tokens = int(ctx.sum())
    algo_bytes = tokens * per_tok + 2 * len(ctx) * 32 * 128 * 2 + ws[0]["tables"].numel() * 4
    ms = timed(torch, step, steps, warmup)
    kms = kernel_ms(torch, L, step, max(20, steps))
    res = dict(metric="tq-t4nc paged-decode attn GB/s" if workload == "decode4" else f"{workload} paged-decode attn GB/s",
               value=algo_bytes / ms / 1e6, ms_per_step=ms,
               dtype="f32 (vector kernels, no matrix cores)" if bits == "tq25" else DECODE_DTYPE,
               config={"workload": name, "context_tokens": tokens, "algorithmic_bytes_per_step": algo_bytes,
                       "cache_copies_alternated": 2, "preconditioning_s": PRECONDITION_S})
    achieved = tokens * per_tok / kms / 1e6
    roof = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            **traffic_fields(workload), "kernel": "main decode-attention kernel", "kernel_ms": kms,
            "algorithmic_bytes_per_launch": tokens * per_tok}
    cpu_obj = None
    if cpu and bits in ("tq35", "tq25"):
        toks, secs, what = cpu_hybrid_baseline(ws[0], tq, cpu_seconds)
        cpu_obj = {"value": toks * per_tok / secs / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
                   "sample": f"numpy float32 oracle (hybrid_decode of every addressed row, dense softmax "
                             f"attention) on {what} = {toks} context tokens"}
    elif cpu:
        toks, secs, seqs = cpu_attention_baseline(ws[0], tq, bits, cpu_seconds)
        cpu_obj = {"value": toks * per_tok / secs / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
                   "sample": f"numpy float32 oracle (gather, unpack, codebook, einsum, softmax, einsum, inverse "
                             f"rotation) on whole sequences {seqs} of the batch = {toks} context tokens"}
        per_tok_s, n_loop = cpu_attention_loop_form(ws[0], tq, bits)
        cpu_obj["loop_form"] = {"value": per_tok / 8 / per_tok_s / 1e9, "unit": "GB/s", "cores": 1,
                                "us_per_token_and_kv_head": per_tok_s * 1e6,
                                "sample": f"the reference's per-token Python loop (TQPagedAttentionRef.forward as the oracle "
                                          f"restates it) on {n_loop} tokens of the longest sequence, one kv head, four query heads"}
    del ws, calls, attn
    torch.cuda.empty_cache()
    return res, roof, cpu_obj


def run_tri(torch, L, dev, steps, warmup, cpu, cpu_seconds, cores):
    from aitherkvcache_amd.triattention import TriAttention, TriAttentionConfig
    cfg = TriAttentionConfig(head_dim=128, num_freqs=12, coeff_bits=4, num_kv_heads=8, num_query_heads=32,
                             rope_base=1e6)
    tri = TriAttention(cfg, device=str(dev))
    gen = torch.Generator(device=dev).manual_seed(4)
    B, S = 8, 32768
    std = (torch.arange(64, device=dev) + 1.0) ** -0.75
    sets = []
    for i in range(3):     # three copies alternated: one copy (109 MB) would sit in the last-level cache
        keys = (torch.randn(B, S, 8, 64, 2, device=dev, generator=gen) * std[:, None]).reshape(B, S, 8, 128).half()
        vals = torch.randn(B, S, 8, 128, device=dev, generator=gen).half()
        sets.append(tri.encode_kv(keys, vals))
        if i == 2:         # the write side: keys and values of the whole batch through the spectral encoder (two launches)
            enc_ms = timed(torch, lambda: tri.encode_kv(keys, vals), 10, 3)
        del keys, vals
    # queries in the model's dtype (fp16, like the keys and values of this configuration); the same step with
    # float32 queries is reported beside it
    q32 = torch.randn(B, 32, 128, device=dev, generator=gen)
    q = q32.half()
    state = {"i": 0, "q": q}

    def step():
        k_enc, v_enc = sets[state["i"] % 3]
        tri.decode_step(state["q"], k_enc, v_enc)
        state["i"] += 1

    algo_bytes = B * S * 8 * 52
    ms = timed(torch, step, steps, warmup)
    kms = kernel_ms(torch, L, step, max(20, steps))
    state["q"] = q32
    kms32 = kernel_ms(torch, L, step, max(20, steps))
    state["q"] = q
    res = dict(metric="TriAttention decode_step GB/s", value=algo_bytes / ms / 1e6, ms_per_step=ms,
               dtype="f32 scores and softmax, fp16 hi/lo MFMA operands for the value sums",
               config={"workload": "config 4: TriAttention decode_step, F=12 int4, 32Q/8KV d=128, batch 8 x 32768, "
                                   "fp16 queries, seed 4",
                       "algorithmic_bytes_per_step": algo_bytes, "cache_copies_alternated": 3,
                       "preconditioning_s": PRECONDITION_S, "kernel_ms_float32_queries": kms32,
                       "encoder_ms": enc_ms, "encoder_vectors": 2 * B * S * 8})
    achieved = algo_bytes / kms / 1e6
    roof = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            **traffic_fields("tri"), "kernel": "tri_decode_heads_kernel<4>", "kernel_ms": kms,
            "algorithmic_bytes_per_launch": algo_bytes}
    cpu_obj = None
    if cpu:
        from oracle import tq_oracle as O
        k_enc, v_enc = sets[0]
        S_s = 2048
        ke = tuple(t[:1, :S_s].cpu().numpy() for t in k_enc)
        ve = tuple(t[:1, :S_s].cpu().numpy() for t in v_enc)
        th = tri._theta.cpu().numpy()
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < cpu_seconds or reps < 1:
            O.tri_decode_step(q[:1].cpu().numpy(), ke, ve, th)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        cpu_obj = {"value": S_s * 8 * 52 / dt / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
                   "sample": f"numpy oracle of decode_step on batch element 0, first {S_s} tokens"}
    del sets
    torch.cuda.empty_cache()
    return res, roof, cpu_obj


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one MI355X: this build has no multi-GPU path (the hot path shards "
              "without communication by sequence, KV head or layer); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    import aitherkvcache_amd as akv
    from aitherkvcache_amd import _lib

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a HIP device")
    dev = torch.device("cuda:0")
    L = _lib.lib()
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    cpu = not args.no_cpu

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    enc, tq4 = bench_encode(torch, akv, L, dev, args.steps, args.warmup, cpu, args.cpu_seconds, sweep=not args.no_sweep)
    out = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "data": "synthetic", "unit": "GB/s"}
    cpu_obj = None

    if args.workload in ("decode4", "decode4_b256", "decode3", "decode2", "tq35", "tq25"):
        res, roof, cpu_obj = run_decode(torch, akv, L, dev, args.workload, tq4, args.steps, args.warmup, cpu,
                                        args.cpu_seconds, cores)
        out.update(res)
        out["roofline"] = roof
    elif args.workload == "tri":
        res, roof, cpu_obj = run_tri(torch, L, dev, args.steps, args.warmup, cpu, args.cpu_seconds, cores)
        out.update(res)
        out["roofline"] = roof
    else:  # encode as the measured step
        n = enc["vectors"]
        out.update(metric="tq-t4nc encode GB/s", value=n * 324 / (n / enc["mvec_s"] / 1e3) / 1e6,
                   ms_per_step=n / enc["mvec_s"] / 1e3,
                   dtype="fp16 input x fp16 hi+lo rotation on MFMA, f32 accumulate, f32 norm and search",
                   config={"workload": "TurboQuant.encode of 2**20 fp16 vectors x 128 (324 B per vector)",
                           "preconditioning_s": PRECONDITION_S})
        out["roofline"] = {"bound": "hbm", "achieved": enc["kernel_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": enc["kernel_frac_hbm"], **traffic_fields("encode"), "kernel": "encode kernel"}
        if cpu:
            cpu_obj = {"value": enc.get("cpu_mvec_s", 0) * 324 / 1e3, "unit": "GB/s", "cores": cores, "kind": "port",
                       "sample": "numpy oracle encode of 65,536 vectors (config 0)"}
    out["cpu_baseline"] = cpu_obj
    out["encode"] = enc
    if args.workload == "decode4" and not args.no_secondary:
        # the other benchmark configurations, same method (two or three cache copies alternated, sustained
        # clocks, kernel time from dispatch time stamps), no CPU leg
        sec = {}
        for wl in ("decode3", "decode2", "tq35", "tq25"):
            r, roof, _ = run_decode(torch, akv, L, dev, wl, tq4, args.steps, args.warmup, False, 0.0, cores)
            sec[wl] = {"workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"], "step_gbs": r["value"],
                       "kernel_ms": roof["kernel_ms"], "algorithmic_bytes_per_launch": roof["algorithmic_bytes_per_launch"],
                       "frac": roof["frac"], "traffic": roof["traffic"], "traffic_source": roof["traffic_source"]}
        r, roof, _ = run_tri(torch, L, dev, args.steps, args.warmup, False, 0.0, cores)
        sec["tri"] = {"workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"], "step_gbs": r["value"],
                      "kernel_ms": roof["kernel_ms"], "kernel_ms_float32_queries": r["config"]["kernel_ms_float32_queries"],
                      "encoder_ms": r["config"]["encoder_ms"], "encoder_vectors": r["config"]["encoder_vectors"],
                      "algorithmic_bytes_per_launch": roof["algorithmic_bytes_per_launch"], "frac": roof["frac"],
                      "traffic": roof["traffic"], "traffic_source": roof["traffic_source"]}
        out["secondary"] = sec
    if not args.no_sweep:
        out["hbm_reference"] = hbm_reference(torch, dev, L)
    print(json.dumps(out))


if __name__ == "__main__":
    main()

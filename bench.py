#!/usr/bin/env python3
"""Benchmark of the ragged paged attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--all]

A *step* is one pass of the hot path over one synthetic batch already resident
in HBM: ``rpa_decode`` (split-KV kernel + combine) on the decode rows followed
by ``rpa_prefill`` (flash kernel) on the prefill rows -- exactly what
``rpa_attention`` issues.  The default workload is the mixed Llama-3-8B batch
(the configuration the headline metric is quoted on).

One JSON line is printed:
  value       decode HBM GB/s of the workload's decode rows: algorithmic bytes /
              measured time of the decode partition (split-KV + combine)
  prefill_tflops, decode_frac_of_hbm_peak, prefill_frac_of_mfma_peak
  roofline    the workload's dominant kernel (largest average launch time),
              timed with events on the launch stream over the timed region
  parity_sample  a few rows of the timed output against the CPU oracle (outside the timed region)
  other_configs  the remaining configurations (C1, C3, C4, C4 windowed, C5), each with its kernel,
              average / median / minimum launch time, algorithmic bytes or FLOPs and roofline fraction
              (--main-only skips them); roofline.configs repeats kernel time and fractions of each, compactly
  ceilings    what this device delivers to the simplest kernels of the same shape, measured in this run: a
              streaming read (contiguous and through a random table of 256 KiB pages) and a matrix-instruction
              issue loop at two waves per SIMD; every roofline object carries frac (of the published peak) and
              frac_of_achievable (of these)
  settle_ms   untimed steps of the same workload run before the warm-up so that the device's clocks have
              left their idle state when the W warm-up and K timed steps start (--settle-ms 0 switches it off)
  host_path   host microseconds per rpa_attention call and per plan-only call, and C1's device time per call
              inside one HIP graph (its latency figure: C1 is bound by launches, not by bytes)
  cpu_baseline  the CPU oracle timed on this box's host cores on a bounded sample

The reference's published perf-guard workloads (32 rows) go to stderr as a JSON line of their own; the line on
stdout keeps their summary.
"""

from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0

# HBM bytes per launch (read + write) of the dominant kernels, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE scaled
# by a 1 GiB device copy (profiles/hbm_traffic_pmc.txt).  Counter runs cannot be taken inside this process, so the
# figures come from sglang-jax_amd/measured_traffic.json, written next to that profile together with the hash of
# the kernel sources they were measured on: when the sources have changed since, `traffic` is null rather than stale.
# kernel that streams the KV bytes of each workload's decode rows: ragged batches that need
# splitting take the balanced plan, equal-length and tiny ones the fixed split plan
DECODE_KERNEL = {
    "c5p": "rpa_mla_decode_wide_kernel",
    "c1": "rpa_decode_splitkv_kernel",
    "c2": "rpa_decode_balanced_kernel",
    "c3": "rpa_decode_splitkv_kernel",
    "c4": "rpa_decode_balanced_kernel",
    "c4swa": "rpa_decode_splitkv_kernel",
    "c5": "rpa_mla_balanced_wide_kernel",
    "c5fp8": "rpa_mla_balanced_kernel",
    "c5tp8": "rpa_mla_balanced_kernel (shared tiles)",
}

PREFILL_KERNEL = "rpa_prefill_pipe_kernel"


def _load_measured_traffic():
    path = os.path.join(ROOT, "sglang-jax_amd", "measured_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f)
        import __graft_entry__ as graft

        if rec.get("source_hash") != graft._load_build_module().source_hash():
            return {}, "the kernel sources changed since profiles/hbm_traffic_pmc.txt was taken"
        return {tuple(k.split("|")): v for k, v in rec["bytes"].items()}, None
    except (OSError, ValueError, KeyError) as e:
        return {}, f"no counter record ({e.__class__.__name__})"


MEASURED_TRAFFIC_BYTES, TRAFFIC_NOTE = _load_measured_traffic()


def _events(n):
    import torch

    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _stats(ms):
    ms = sorted(ms)
    n = len(ms)
    return {"mean": sum(ms) / n, "median": ms[n // 2] if n % 2 else 0.5 * (ms[n // 2 - 1] + ms[n // 2]), "min": ms[0]}


def settle(step, ms):
    """Untimed steps for about `ms` milliseconds of wall time (at most 2000 steps): a device that starts from
    idle runs its first milliseconds at other clocks than the rest.  Returns what it did."""
    import torch

    if ms <= 0:
        return {"ms": 0.0, "steps": 0}
    torch.cuda.synchronize()
    t0, n = time.perf_counter(), 0
    while (time.perf_counter() - t0) * 1e3 < ms and n < 2000:
        for _ in range(5):
            step()
        n += 5
        torch.cuda.synchronize()
    return {"ms": (time.perf_counter() - t0) * 1e3, "steps": n}


def _series(ms):
    """Per-step durations of the timed region in microseconds, in step order, with the means of the first and
    the last quarter: a drift over the region (clocks, caches) shows here."""
    q = max(1, len(ms) // 4)
    return {"us": [round(x * 1e3, 1) for x in ms], "first_quarter_mean_us": sum(ms[:q]) / q * 1e3,
            "last_quarter_mean_us": sum(ms[-q:]) / q * 1e3}


def time_partitions(call, steps, warmup, has_decode, has_prefill, settle_ms=0.0):
    """`settle_ms` of untimed steps, W warm-up steps, then exactly `steps` timed steps; returns wall ms per
    step and mean / median / min of the event-timed duration of each partition inside the timed region."""
    import torch

    def one(ev=None):
        if ev is not None:
            ev[0].record()
        if has_decode:
            call.decode()
        if ev is not None:
            ev[1].record()
        if has_prefill:
            call.prefill()
        if ev is not None:
            ev[2].record()

    settled = settle(one, settle_ms)
    for _ in range(warmup):
        one()
    evs = [_events(3) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        one(evs[i])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    dec_ms = [e[0].elapsed_time(e[1]) for e in evs]
    pre_ms = [e[1].elapsed_time(e[2]) for e in evs]
    dec, pre = _stats(dec_ms), _stats(pre_ms)
    dec["series"], pre["series"] = _series(dec_ms), _series(pre_ms)
    dec["settle"] = pre["settle"] = settled
    # After the timed region: each partition again as `steps` launches in a row between ONE pair of
    # events.  An event recorded between two kernels is a packet of its own that the next kernel
    # waits for, so the per-step figures above carry a few microseconds of the measurement itself;
    # this figure does not, and is the one to hold against a profiler's per-kernel durations.
    def stream(fn):
        a, b = _events(2)
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / steps

    if has_decode:
        dec["back_to_back"] = stream(call.decode)
    if has_prefill:
        pre["back_to_back"] = stream(call.prefill)
    return (t1 - t0) * 1e3 / steps, dec, pre


def make_call(pkg, b, static_shapes=False):
    import numpy as np

    m = importlib.import_module("sglang_jax_amd.ragged_paged_attention")
    n = int(b.distribution[2])
    q_lens = b.q_lens()[:n]
    dec_end = int(b.distribution[0])
    if static_shapes:
        # nothing but static shapes on the host: the kernels read the composition from the device
        return m.RpaCall(b.q, b.kv_cache, None, b.kv_lens, b.page_indices, b.cu_q_lens, b.cu_kv_lens,
                         num_seqs=int(b.kv_lens.shape[0]), decode_end=0, sm_scale=b.sm_scale,
                         sliding_window=b.sliding_window, soft_cap=b.soft_cap, k_scale=b.k_scale, v_scale=b.v_scale,
                         max_q_len=2048 if n > dec_end else 0,  # the workload's chunk size: a static bound, like chunk_prefill_size
                         distribution_d=b.distribution)
    return m.RpaCall(b.q, b.kv_cache, None, b.kv_lens, b.page_indices, b.cu_q_lens, b.cu_kv_lens, num_seqs=n,
                     decode_end=dec_end, sm_scale=b.sm_scale, sliding_window=b.sliding_window, soft_cap=b.soft_cap,
                     k_scale=b.k_scale, v_scale=b.v_scale, max_kv_len=int(max(b.meta["kv_lens"])),
                     max_q_len=int(q_lens[dec_end:].max()) if n > dec_end else 0,
                     sum_decode_kv_len=int(sum(b.meta["kv_lens"][:dec_end])))


def run_rpa_config(pkg, wl, b, steps, warmup, keep_call=False, static_shapes=False, settle_ms=0.0, series=False):
    dec_end, n = int(b.distribution[0]), int(b.distribution[2])
    call = make_call(pkg, b, static_shapes)
    ms, dec, pre = time_partitions(call, steps, warmup, dec_end > 0, n > dec_end, settle_ms)
    res = {"workload": b.name, "ms_per_step": ms, "settle": dec["settle"]}
    if series:
        if dec_end > 0:
            res["decode_series"] = dec["series"]
        if n > dec_end:
            res["prefill_series"] = pre["series"]
    if dec_end > 0:
        nbytes = wl.decode_bytes(b, 0, dec_end)
        res.update(decode_ms=dec["mean"], decode_ms_median=dec["median"], decode_ms_min=dec["min"], decode_bytes=nbytes,
                   decode_gbps=nbytes / (dec["mean"] * 1e-3) / 1e9, decode_ms_back_to_back=dec["back_to_back"],
                   decode_gbps_back_to_back=nbytes / (dec["back_to_back"] * 1e-3) / 1e9)
    if n > dec_end:
        flops = wl.prefill_flops(b, dec_end, n)
        res.update(prefill_ms=pre["mean"], prefill_ms_median=pre["median"], prefill_ms_min=pre["min"],
                   prefill_flops=flops, prefill_tflops=flops / (pre["mean"] * 1e-3) / 1e12,
                   prefill_ms_back_to_back=pre["back_to_back"],
                   prefill_tflops_back_to_back=flops / (pre["back_to_back"] * 1e-3) / 1e12)
    return (res, call) if keep_call else res


def parity_sample(wl, b, call):
    """A few rows of the output the timed steps left behind against the CPU oracle: the first, the
    longest and the last decode row and the last 128 rows of the last chunk, re-run by the oracle on
    a compact copy of their pages.  Outside the timed region."""
    import numpy as np
    import torch

    from oracle.ref_rpa import ref_ragged_paged_attention_fused

    dec_end, n = int(b.distribution[0]), int(b.distribution[2])
    kv = np.asarray(b.meta["kv_lens"])
    seqs = sorted({0, int(np.argmax(kv[:dec_end])), dec_end - 1}) if dec_end > 0 else []
    if n > dec_end:
        seqs.append(n - 1)
    sample = wl.sub_batch(b, seqs, last_rows=128)
    want = ref_ragged_paged_attention_fused(sample.q, sample.kv_cache, sample.kv_lens, sample.padded_page_table(),
                                            sample.cu_q_lens, [len(seqs)], sm_scale=sample.sm_scale,
                                            sliding_window=sample.sliding_window, soft_cap=sample.soft_cap,
                                            k_scale=sample.k_scale, v_scale=sample.v_scale).float()
    torch.cuda.synchronize()
    got = call.out[torch.tensor(sample.meta["rows"], device=call.out.device)].float().cpu()
    rel = ((got - want).norm(dim=-1) / want.norm(dim=-1).clamp_min(1e-30)).max()
    return {"sequences": seqs, "rows": int(got.shape[0]), "max_abs_err": float((got - want).abs().max()),
            "max_row_rel_err": float(rel), "tolerance": "rtol = atol = 2e-2 (5e-2 fp8 KV), row-relative 1e-2 (3e-2)"}


def run_mla_config(pkg, wl, b, steps, warmup, settle_ms=0.0):
    import torch

    n = int(b.distribution[2])
    kw = dict(sm_scale=b.sm_scale, max_kv_len=int(max(b.meta["kv_lens"])), sum_kv_len=int(sum(b.meta["kv_lens"])))
    dist = b.distribution.cpu().numpy()

    def one():
        pkg.mla_ragged_paged_attention(b.ql_nope, b.q_pe, None, None, b.cache_kv, b.kv_lens, b.page_indices,
                                       b.cu_q_lens, b.cu_kv_lens, dist, **kw)

    settled = settle(one, settle_ms)
    for _ in range(warmup):
        one()
    evs = [_events(2) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for e in evs:
        e[0].record()
        one()
        e[1].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    st = _stats([e[0].elapsed_time(e[1]) for e in evs])
    ms = st["mean"]
    if any(q != 1 for q in b.meta["q_lens"]):  # prefill chunks: a FLOP figure, no decode bytes
        flops = wl.mla_attention_flops(b)
        return {"workload": b.name, "ms_per_step": (t1 - t0) * 1e3 / steps, "settle": settled, "prefill_ms": ms, "prefill_ms_median": st["median"],
                "prefill_ms_min": st["min"], "prefill_flops": flops, "prefill_tflops": flops / (ms * 1e-3) / 1e12}
    nbytes, flops = wl.mla_decode_bytes(b), wl.mla_decode_flops(b)
    return {"workload": b.name, "ms_per_step": (t1 - t0) * 1e3 / steps, "settle": settled, "decode_ms": ms, "decode_ms_median": st["median"],
            "decode_ms_min": st["min"], "decode_bytes": nbytes, "decode_gbps": nbytes / (ms * 1e-3) / 1e9,
            "tflops": flops / (ms * 1e-3) / 1e12}


# The reference's own published figures for this path: the perf-guard baselines of its TPU kernel
# (benchmark/kernels/flash_attention/bench_flashattention.py:264-328; device time of the op in ms,
# bf16, head_dim 128, 600 000-token pool; heads are per device).  key: (mode, page_size, tokens or
# batch, q heads, kv heads) -> (TPU v6e, TPU v7).
REFERENCE_PUBLISHED_MS = {
    ("prefill", 128, 1024, 4, 1): (0.0334175, 0.014767107), ("prefill", 128, 1024, 4, 2): (0.05767375, 0.015102041),
    ("prefill", 128, 1024, 8, 1): (0.04415, 0.022470588), ("prefill", 128, 1024, 8, 4): (0.0835275, 0.023110444),
    ("prefill", 128, 4096, 4, 1): (0.19460875, 0.0794994), ("prefill", 128, 4096, 4, 2): (0.34417875, 0.084321729),
    ("prefill", 128, 4096, 8, 1): (0.25254875, 0.145336134), ("prefill", 128, 4096, 8, 4): (0.50654375, 0.145752701),
    ("prefill", 256, 1024, 4, 1): (0.03286125, 0.014686675), ("prefill", 256, 1024, 4, 2): (0.0571225, 0.015236495),
    ("prefill", 256, 1024, 8, 1): (0.043765, 0.022472989), ("prefill", 256, 1024, 8, 4): (0.0829025, 0.023372149),
    ("prefill", 256, 4096, 4, 1): (0.19131, 0.079831933), ("prefill", 256, 4096, 4, 2): (0.34008, 0.084252101),
    ("prefill", 256, 4096, 8, 1): (0.25009625, 0.144997599), ("prefill", 256, 4096, 8, 4): (0.50262875, 0.145212485),
    ("decode", 128, 128, 4, 1): (0.58231125, 0.15942617), ("decode", 128, 128, 4, 2): (0.3259175, 0.226237695),
    ("decode", 128, 128, 8, 1): (0.5799825, 0.159394958), ("decode", 128, 128, 8, 4): (0.55449, 0.331831933),
    ("decode", 128, 256, 4, 1): (1.1546875, 0.313444178), ("decode", 128, 256, 4, 2): (0.64474375, 0.452889556),
    ("decode", 128, 256, 8, 1): (1.150025, 0.313991597), ("decode", 128, 256, 8, 4): (1.1009563, 0.649698679),
    ("decode", 256, 128, 4, 1): (0.54297, 0.15329892), ("decode", 256, 128, 4, 2): (0.28788125, 0.207255702),
    ("decode", 256, 128, 8, 1): (0.5406875, 0.152806723), ("decode", 256, 128, 8, 4): (0.42053875, 0.313996399),
    ("decode", 256, 256, 4, 1): (1.0762225, 0.303966387), ("decode", 256, 256, 4, 2): (0.56767875, 0.415367347),
    ("decode", 256, 256, 8, 1): (1.0714862, 0.303222089), ("decode", 256, 256, 8, 4): (None, 0.610410564),
}


def reference_suite(pkg, wl, dev, reps=50):
    """The reference's perf-guard workloads on this GPU, timed the way its harness times them: device time
    of the whole op, new-token cache write included (its kernel fuses the write; here rpa_kv_write +
    rpa_attention).  Prefill = N tokens cut into 2048-token sequences with q_len == kv_len
    (benchmark/kernels/flash_attention/utils.py:61-68, bench_flashattention.py:59-62); decode = N rows of one
    token on 1025..2048 cached tokens (utils.py:131-132; numpy draws here, jax draws there).  `reps` steps are
    captured in ONE HIP graph so that the figure is kernels back to back, not launch overhead."""
    import numpy as np
    import torch

    m = importlib.import_module("sglang_jax_amd.ragged_paged_attention")
    rows = []
    for (mode, P, N, Hq, Hkv), (v6e, v7) in REFERENCE_PUBLISHED_MS.items():
        if mode == "prefill":
            q_lens = [2048] * (N // 2048) + ([N % 2048] if N % 2048 else [])
            kv_lens = list(q_lens)
        else:
            kv_lens = (np.random.default_rng(42).integers(1024, 2048, size=N) + 1).tolist()
            q_lens = [1] * N
        b = wl.make_batch(f"reference_{mode}", q_lens, kv_lens, num_q_heads=Hq, num_kv_heads=Hkv, head_dim=128,
                          page_size=P, seed=42, device=dev, pool_pages=600000 // P)
        T, n = sum(q_lens), len(q_lens)
        dec = n if mode == "decode" else 0
        keys = torch.randn(T, Hkv, 128, device=dev, dtype=torch.bfloat16)
        vals = torch.randn(T, Hkv, 128, device=dev, dtype=torch.bfloat16)
        call = m.RpaCall(b.q, b.kv_cache, None, b.kv_lens, b.page_indices, b.cu_q_lens, b.cu_kv_lens, num_seqs=n,
                         decode_end=dec, sm_scale=b.sm_scale, max_kv_len=max(kv_lens), max_q_len=max(q_lens),
                         sum_decode_kv_len=sum(kv_lens) if dec else 0, own_workspace=True)

        def step():
            call.kv_write(keys, vals)
            call.attention()

        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(reps):
                step()
        graph.replay()
        torch.cuda.synchronize()
        e0, e1 = _events(2)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        rows.append({"mode": mode, "page_size": P, "tokens_or_batch": N, "q_heads": Hq, "kv_heads": Hkv, "ms": ms,
                     "tpu_v6e_ms": v6e, "tpu_v7_ms": v7, "speedup_vs_v6e": None if v6e is None else v6e / ms,
                     "speedup_vs_v7": v7 / ms})
        del call, b, keys, vals, graph
    return rows


def measure_ceilings(dev, nbytes=2 << 30, reps=5):
    """What this device delivers to the simplest kernels of the attention kernels' shape (csrc/rpa_ceilings.hip,
    lib/librpa_ceilings.so), event-timed on the current stream:
      * a streaming read of `nbytes` of random data, every wave sixteen 16-byte loads per lane in flight, over
        wave counts from 3.5 per CU (the decode plan's: 4) to 32 per CU, contiguous and through a random table of
        256 KiB pages (one page = 64 tokens of 8 kv heads x 128 dims, bf16 K and V), each wave on a contiguous
        run of blocks or the waves interleaved block by block, with plain and with non-temporal loads (the
        decode kernels' kind);
      * v_mfma_f32_32x32x16_bf16 into four independent accumulators, two waves per SIMD.
    `achievable` holds the best of each: the denominators of frac_of_achievable."""
    import ctypes

    import torch

    path = os.path.join(ROOT, "sglang-jax_amd", "lib", "librpa_ceilings.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is not built: run __graft_entry__.build()")
    lib = ctypes.CDLL(path)
    lib.rpa_ceiling_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64,
                                            ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.rpa_ceiling_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.rpa_ceiling_lds_dma_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                             ctypes.c_void_p]
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    page_bytes = 256 << 10
    src = torch.empty(nbytes // 8, dtype=torch.int64, device=dev).random_()
    table = torch.randperm(nbytes // page_bytes, generator=torch.Generator().manual_seed(7)).to(torch.int32).to(dev)
    sink = torch.zeros(64, dtype=torch.int32, device=dev)

    def timed(launch, n):
        for _ in range(2):
            launch()
        a, b = _events(2)
        a.record()
        for _ in range(n):
            launch()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n

    rows = []
    plan_waves = cus * 4  # the decode plan's resident waves on long rows (one per SIMD)
    for waves in (cus * 4 - cus // 2, plan_waves, cus * 8, cus * 16, cus * 32):
        for order in (0, 1):
            for paged in (False, True):
                for nt in (False, True):
                    def launch():
                        rc = lib.rpa_ceiling_stream_read(src.data_ptr(), nbytes, table.data_ptr() if paged else None, page_bytes,
                                                         waves, order + (4 if nt else 0), sink.data_ptr(), stream)
                        if rc != 0:
                            raise RuntimeError(f"rpa_ceiling_stream_read: hip error {rc}")
                    ms = timed(launch, reps)
                    rows.append({"waves": waves, "order": "contiguous runs" if order == 0 else "interleaved", "paged": paged,
                                 "loads": "non-temporal" if nt else "plain", "ms": ms, "gbps": nbytes / (ms * 1e-3) / 1e9})
    # the same contiguous stream moved into LDS by global_load_lds_dwordx4 (how the prefill and MLA kernels fill their
    # tile rings), one workgroup of four waves per CU
    dma_rows = []
    for nt in (False, True):
        def launch_dma():
            rc = lib.rpa_ceiling_lds_dma_read(src.data_ptr(), nbytes, cus * 4, 1 if nt else 0, sink.data_ptr(), stream)
            if rc != 0:
                raise RuntimeError(f"rpa_ceiling_lds_dma_read: hip error {rc}")
        ms = timed(launch_dma, reps)
        dma_rows.append({"waves": cus * 4, "loads": "non-temporal" if nt else "plain", "ms": ms, "gbps": nbytes / (ms * 1e-3) / 1e9})
    iters = 2000
    wgs = 2 * cus

    def launch_mfma():
        rc = lib.rpa_ceiling_mfma(wgs, iters, sink.data_ptr(), stream)
        if rc != 0:
            raise RuntimeError(f"rpa_ceiling_mfma: hip error {rc}")
    mfma_ms = timed(launch_mfma, reps)
    mfma_tflops = wgs * 4 * iters * 16 * 32768 / (mfma_ms * 1e-3) / 1e12
    best = lambda paged, waves=None: max(r["gbps"] for r in rows if r["paged"] == paged and (waves is None or r["waves"] == waves))
    del src, table
    torch.cuda.empty_cache()
    return {
        "what": "streaming read of %d MiB (16 KiB per wave in flight) and a v_mfma_f32_32x32x16_bf16 issue loop at two "
                "waves per SIMD, measured in this run" % (nbytes >> 20),
        "achievable": {"hbm_read_gbps_contiguous": best(False), "hbm_read_gbps_paged_256KiB": best(True),
                       "hbm_read_gbps_paged_at_decode_plan_waves": best(True, plan_waves),
                       "hbm_read_gbps_plain_loads": max(r["gbps"] for r in rows if r["loads"] == "plain"),
                       "hbm_read_gbps_non_temporal_loads": max(r["gbps"] for r in rows if r["loads"] == "non-temporal"),
                       "hbm_read_gbps_into_lds_plain": dma_rows[0]["gbps"],
                       "hbm_read_gbps_into_lds_non_temporal": dma_rows[1]["gbps"],
                       "mfma_bf16_tflops": mfma_tflops},
        "frac_of_published_peak": {"hbm_contiguous": best(False) / HBM_PEAK_GBPS, "hbm_paged": best(True) / HBM_PEAK_GBPS,
                                   "mfma_bf16": mfma_tflops / MFMA_BF16_PEAK_TFLOPS},
        "mfma_loop_ms": mfma_ms, "stream_read": rows, "stream_read_into_lds": dma_rows,
    }


def host_path(pkg, wl, dev, calls=2000, reps=50):
    """What the host side of a call costs, on the latency-bound configuration (C1: 8 decode rows, 14 us of GPU
    work): microseconds of host time per rpa_attention through the C ABI (ctypes included; the queue is drained
    first and the loop is short enough not to fill it), the same for the plan arithmetic alone
    (rpa_workspace_bytes: shape table, split plan, no launch), and the device time per call when `reps` calls
    are replayed as one HIP graph (kernels back to back, no host in between)."""
    import ctypes

    import torch

    b = wl.config_c1(dev)
    call = make_call(pkg, b)
    lib = pkg._lib.load()
    for _ in range(20):
        call.attention()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(calls):
        call.attention()
    t1 = time.perf_counter()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    pp = ctypes.byref(call.params)
    t3 = time.perf_counter()
    for _ in range(calls):
        lib.rpa_workspace_bytes(pp)
    t4 = time.perf_counter()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        for _ in range(3):
            call.attention()
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(reps):
            call.attention()
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = _events(2)
    e0.record()
    graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return {"workload": b.name, "host_us_per_rpa_attention": (t1 - t0) * 1e6 / calls,
            "wall_us_per_call_drained": (t2 - t0) * 1e6 / calls,
            "host_us_per_plan_only_call": (t4 - t3) * 1e6 / calls,
            "device_us_per_call_in_one_graph": e0.elapsed_time(e1) * 1e3 / reps, "calls": calls, "graph_calls": reps}


def cpu_baseline(wl, budget_s=10.0, prefill_budget_s=8.0):
    """CPU oracle on a bounded sample of the default workload: its first decode rows
    (same seeded lengths and layout, values drawn on the host), and -- reported under `prefill` -- one
    256-token chunk on a 512-token prefix with the same heads."""
    import torch

    from oracle.ref_rpa import ref_ragged_paged_attention_fused

    import numpy as np

    rng = np.random.Generator(np.random.PCG64(1002))
    kv_d = rng.integers(512, 4096, size=56, endpoint=True)
    rows = 8
    b = wl.make_batch("c2_decode_rows_0_7", np.ones(rows, int), kv_d[:rows], num_q_heads=32, num_kv_heads=8,
                      head_dim=128, page_size=64, seed=1002)
    table = b.padded_page_table()
    torch.set_num_threads(os.cpu_count() or 1)
    f = lambda: ref_ragged_paged_attention_fused(b.q, b.kv_cache, b.kv_lens, table, b.cu_q_lens, [rows],
                                                 sm_scale=b.sm_scale)
    f()
    reps, t0 = 0, time.perf_counter()
    while True:
        f()
        reps += 1
        if time.perf_counter() - t0 > budget_s or reps >= 1000:
            break
    dt = (time.perf_counter() - t0) / reps
    nbytes = wl.decode_bytes(b)
    # the prefill side of the same workload
    pb = wl.make_batch("c2_prefill_sample", [256], [768], num_q_heads=32, num_kv_heads=8, head_dim=128, page_size=64,
                       seed=1003)
    ptable = pb.padded_page_table()
    g = lambda: ref_ragged_paged_attention_fused(pb.q, pb.kv_cache, pb.kv_lens, ptable, pb.cu_q_lens, [1],
                                                 sm_scale=pb.sm_scale)
    g()
    preps, t1 = 0, time.perf_counter()
    while True:
        g()
        preps += 1
        if time.perf_counter() - t1 > prefill_budget_s or preps >= 200:
            break
    pdt = (time.perf_counter() - t1) / preps
    return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"CPU oracle (torch f32) on decode rows 0..{rows - 1} of c2_llama3_8b_mixed "
                      f"(kv_lens {kv_d[:rows].tolist()}), {reps} reps, {dt * 1e3:.1f} ms each",
            "prefill": {"value": wl.prefill_flops(pb) / pdt / 1e12, "unit": "TFLOP/s",
                        "sample": f"the same oracle on one 256-token chunk on a 512-token prefix (32 / 8 heads of 128), "
                                  f"{preps} reps, {pdt * 1e3:.1f} ms each"}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="c2", choices=["c1", "c2", "c3", "c4", "c4swa", "c5", "c5fp8", "c5tp8", "c5p", "c5p16"],
                    help="c5p: absorbed-MLA prefill chunks (512 tokens on 4096-token prefixes), DeepSeek-V3 shape; "
                         "c5fp8: C5 on an e4m3 latent cache; c5tp8: C5 with 16 of the 128 heads (one GPU's share at tensor-parallel 8); "
                         "c5p16: the c5p chunks with 16 heads, the head count of the reference's own MLA tests")
    ap.add_argument("--all", action="store_true", help="(default) also time the other configurations")
    ap.add_argument("--main-only", action="store_true", help="skip the other configurations")
    ap.add_argument("--reference-suite", action="store_true",
                    help="with --main-only: still run the reference's own perf-guard workloads")
    ap.add_argument("--static-shapes", action="store_true",
                    help="run the main configuration with the batch composition read on the device (grids sized "
                         "from static shapes only)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed steps of the same workload for this many milliseconds before the warm-up (reported "
                         "as settle_ms; 0 = none): the first milliseconds after idle run at other clocks")
    ap.add_argument("--ceilings", action="store_true",
                    help="only measure what the device delivers to a plain streaming read and to a matrix-instruction "
                         "issue loop (the denominators of frac_of_achievable) and print them")
    ap.add_argument("--no-ceilings", action="store_true", help="skip those measurements (no frac_of_achievable)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 1 GiB device-to-device copy (10 launches): the known-size kernel "
                         "against which rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no sharding, no collectives); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import __graft_entry__ as graft

    graft.ensure_built()
    pkg = graft.load_package()
    wl = importlib.import_module("sglang_jax_amd.workloads")
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the operators have no CPU path", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4, "launches": 10}))
        return

    if args.ceilings:
        print(json.dumps({"ceilings": measure_ceilings(dev, reps=10)}))
        return
    ceilings = None if args.no_ceilings else measure_ceilings(dev)

    def achievable(bound):
        if ceilings is None:
            return None
        return ceilings["achievable"]["hbm_read_gbps_paged_256KiB" if bound == "hbm" else "mfma_bf16_tflops"]

    def with_achievable(r):
        """frac_of_achievable next to frac: the same figure against what a plain kernel reaches on this device"""
        top = achievable(r["bound"])
        if TRAFFIC_NOTE and "traffic" in r:
            r["traffic_note"] = TRAFFIC_NOTE
        r["frac_of_achievable"] = None if top is None else r["achieved"] / top
        if r.get("frac_back_to_back") is not None and top is not None:
            r["frac_of_achievable_back_to_back"] = r["frac_back_to_back"] * r["peak"] / top
        return r

    def build(name):
        return {"c1": lambda: wl.config_c1(dev), "c2": lambda: wl.config_c2(dev), "c3": lambda: wl.config_c3(dev),
                "c4": lambda: wl.config_c4(dev), "c4swa": lambda: wl.config_c4(dev, window=True),
                "c5": lambda: wl.config_c5(dev), "c5p": lambda: wl.config_c5_prefill(dev),
                "c5fp8": lambda: wl.config_c5(dev, kv_dtype=torch.float8_e4m3fn),
                "c5tp8": lambda: wl.config_c5(dev, num_q_heads=16),
                "c5p16": lambda: wl.config_c5_prefill(dev, num_q_heads=16)}[name]()

    def run(name, keep=False):
        b = build(name)
        if name in ("c5", "c5p", "c5fp8", "c5tp8", "c5p16"):
            r = run_mla_config(pkg, wl, b, args.steps, args.warmup, settle_ms=args.settle_ms)
        elif keep:
            r, call = run_rpa_config(pkg, wl, b, args.steps, args.warmup, keep_call=True,
                                     static_shapes=args.static_shapes, settle_ms=args.settle_ms, series=True)
            r = (r, parity_sample(wl, b, call))
            del call
        else:
            r = run_rpa_config(pkg, wl, b, args.steps, args.warmup, settle_ms=args.settle_ms)
        del b
        torch.cuda.empty_cache()
        return r

    def decode_roofline(name, res):
        kernel = DECODE_KERNEL[name]
        rl = {"kernel": kernel + (" + combine" if name != "c1" else ""), "bound": "hbm",
                "achieved": res["decode_gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": res["decode_gbps"] / HBM_PEAK_GBPS, "traffic": MEASURED_TRAFFIC_BYTES.get((name, kernel)),
                "avg_launch_ms": res["decode_ms"], "median_launch_ms": res["decode_ms_median"],
                "min_launch_ms": res["decode_ms_min"], "bytes_per_launch": res["decode_bytes"],
                "back_to_back_launch_ms": res.get("decode_ms_back_to_back"),
                "frac_back_to_back": (res["decode_gbps_back_to_back"] / HBM_PEAK_GBPS
                                      if "decode_gbps_back_to_back" in res else None)}
        if name == "c5fp8":
            # 128 heads on an e4m3 latent cache: 421 FLOP per byte, above the ridge (2.5 PFLOP/s : 8 TB/s = 312)
            rl.update({"bound": "mfma", "achieved": res["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                       "frac": res["tflops"] / MFMA_BF16_PEAK_TFLOPS, "hbm_frac": res["decode_gbps"] / HBM_PEAK_GBPS,
                       "frac_back_to_back": None})
        return rl

    if args.config in ("c5", "c5p", "c5fp8", "c5tp8", "c5p16"):
        main_res, sample = run(args.config), None
    else:
        main_res, sample = run(args.config, keep=True)
    dec_gbps = main_res.get("decode_gbps")
    pre_tflops = main_res.get("prefill_tflops")
    # dominant kernel of the workload (largest average launch time inside the timed region)
    roofline_decode = with_achievable(decode_roofline(args.config, main_res)) if dec_gbps is not None else None
    prefill_kernel = {"c5p": "rpa_mla_decode_wide_kernel (one row per query token)",
                      "c5p16": "rpa_mla_token_group_wide_kernel (8 query tokens per workgroup)"}.get(args.config, PREFILL_KERNEL)

    def prefill_roofline(name, res, kernel):
        return with_achievable({
            "kernel": kernel, "bound": "mfma", "achieved": res["prefill_tflops"], "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": res["prefill_tflops"] / MFMA_BF16_PEAK_TFLOPS,
            "traffic": MEASURED_TRAFFIC_BYTES.get((name, kernel)), "avg_launch_ms": res["prefill_ms"],
            "median_launch_ms": res["prefill_ms_median"], "min_launch_ms": res["prefill_ms_min"],
            "flops_per_launch": res["prefill_flops"], "back_to_back_launch_ms": res.get("prefill_ms_back_to_back"),
            "frac_back_to_back": (res["prefill_tflops_back_to_back"] / MFMA_BF16_PEAK_TFLOPS
                                  if "prefill_tflops_back_to_back" in res else None)})

    roofline_prefill = prefill_roofline(args.config, main_res, prefill_kernel) if pre_tflops is not None else None
    if pre_tflops is not None and main_res.get("prefill_ms", 0) >= main_res.get("decode_ms", 0):
        roofline = dict(roofline_prefill)
    else:
        roofline = dict(roofline_decode)
    line = {
        "metric": "ragged paged attn: decode HBM GB/s (% of peak), prefill TFLOP/s; 1 MI355X",
        "value": dec_gbps if dec_gbps is not None else pre_tflops,
        "unit": "GB/s" if dec_gbps is not None else "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_res["ms_per_step"],
        "settle_ms": main_res["settle"]["ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.config not in ("c4", "c4swa", "c5fp8") else "bf16 (fp8-e4m3 KV)", "data": "synthetic",
        "config": {"workload": main_res["workload"], "value_is": "decode partition (split-KV + combine) algorithmic bytes / time",
                   "call_mode": "static shapes, composition read on the device" if args.static_shapes else "host integers",
                   "settle": "%d untimed steps (%.0f ms) before the %d warm-up steps" % (
                       main_res["settle"]["steps"], main_res["settle"]["ms"], args.warmup)},
        "decode_frac_of_hbm_peak": None if dec_gbps is None else dec_gbps / HBM_PEAK_GBPS,
        "prefill_tflops": pre_tflops,
        "prefill_frac_of_mfma_peak": None if pre_tflops is None else pre_tflops / MFMA_BF16_PEAK_TFLOPS,
        "partitions": main_res,
        "roofline": roofline,
        "roofline_decode": roofline_decode,
        "parity_sample": sample,
        "ceilings": ceilings,
    }
    # every configuration's dominant kernel in one compact map inside `roofline`:
    # name -> [kernel, bound, average launch ms, fraction of the published peak, fraction of the achievable]
    compact = lambda r: [r["kernel"], r["bound"], round(r["avg_launch_ms"], 5), round(r["frac"], 4),
                         None if r["frac_of_achievable"] is None else round(r["frac_of_achievable"], 4)]
    configs = {}
    if roofline_decode is not None:
        configs[args.config + (" decode rows" if roofline_prefill is not None else "")] = compact(roofline_decode)
    if roofline_prefill is not None:
        configs[args.config + (" prefill rows" if roofline_decode is not None else "")] = compact(roofline_prefill)
    if not args.main_only:
        others = {}
        for name in ("c1", "c2", "c3", "c4", "c4swa", "c5", "c5fp8", "c5tp8", "c5p", "c5p16"):
            if name == args.config:
                continue
            r = run(name)
            if name in ("c5p", "c5p16"):
                r["roofline"] = with_achievable({
                    "kernel": "rpa_mla_decode_wide_kernel (one row per query token)" if name == "c5p"
                              else "rpa_mla_token_group_wide_kernel (8 query tokens per workgroup)", "bound": "mfma",
                    "achieved": r["prefill_tflops"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": r["prefill_tflops"] / MFMA_BF16_PEAK_TFLOPS, "avg_launch_ms": r["prefill_ms"],
                    "flops_per_launch": r["prefill_flops"]})
                others[name] = r
                configs[name] = compact(r["roofline"])
                continue
            r["roofline"] = with_achievable(decode_roofline(name, r))
            configs[name + (" decode rows" if "prefill_tflops" in r else "")] = compact(r["roofline"])
            if name in ("c5", "c5tp8"):
                r["roofline"]["mfma_frac"] = r["tflops"] / MFMA_BF16_PEAK_TFLOPS
            if "prefill_tflops" in r:
                r["roofline_prefill"] = prefill_roofline(name, r, PREFILL_KERNEL)
                configs[name + " prefill rows"] = compact(r["roofline_prefill"])
            others[name] = r
        line["other_configs"] = others
    roofline["configs"] = configs
    roofline["configs_columns"] = ["kernel", "bound", "avg_launch_ms", "frac", "frac_of_achievable"]
    if args.reference_suite or not args.main_only:
        rows = reference_suite(pkg, wl, dev)
        what = ("the reference's published perf-guard workloads (bench_flashattention.py:264-328), device ms per op "
                "with the new-token cache write, this GPU against its TPU v6e / v7 baselines")
        # the 32 rows go to stderr as a line of their own: stdout holds the one line with the headline
        print(json.dumps({"reference_suite": {"what": what, "rows": rows}}), file=sys.stderr)
        v6 = [r["speedup_vs_v6e"] for r in rows if r["speedup_vs_v6e"] is not None]
        v7 = [r["speedup_vs_v7"] for r in rows]
        line["reference_suite"] = {
            "what": what + "; the rows are on stderr", "workloads": len(rows),
            "speedup_vs_v6e_min_max": [min(v6), max(v6)], "speedup_vs_v7_min_max": [min(v7), max(v7)],
            "ahead_of_v6e": sum(x > 1 for x in v6), "ahead_of_v7": sum(x > 1 for x in v7)}
    if not args.main_only:
        line["host_path"] = host_path(pkg, wl, dev)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(line))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the full-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--main-only] [--no-cpu]

Headline workload (one "step"): one layer's attention core over a 672-token
prompt at depth 0 -- RoPE of Q and K, q8_0 quantize-and-append of K/V, causal
GQA attention over the q8_0 cache (24 query heads, 4 KV heads, head_dim 256),
sigmoid output gate -- with every input already resident in HBM.  Steps rotate
over 16 distinct layer caches.  value = tokens/s of that step.

The same JSON line carries, under "also", the other workloads of the path
(decode at 8,192 / 32,768, the 2,048-token chunk at depth 100,000, batched
decode with MTP-verify slots), each with its own roofline object.

roofline.achieved = algorithmic FLOP (prefill) or K+V cache bytes (decode) per
attention launch / the attention launch's mean duration measured with HIP
events on the launch stream.  roofline.achievable = what a kernel that does
nothing else reaches on this box in the same run: a pure read of the same bytes
in the decode kernel's access pattern, or a loop of independent MFMAs (the
library's measurement-only entry points hipml_bench_*).  Every figure is the mean
over at least --steps steps and at least 200 ms of timed GPU work (the reference
sizes its repetitions the same way, crates/hipml-kernels/src/kvbench.rs:160-163);
`timed_ms` and `steps_timed` say what was timed.  cpu_baseline = the CPU oracle (a
scalar restatement of the reference's CPU path) timed on this host on the stated
sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

H, KV, HD, NROT, THETA = 24, 4, 256, 64, 1e7
ROW = 272
SCALE = 1.0 / 16.0
HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_F16_PEAK_TF = 2500.0  # MI355X dense fp16 MFMA, published
LAYERS = 16                # distinct layer caches a pass rotates over
MIN_TIMED_MS = 200.0       # every figure is a mean over at least this much timed GPU work
MFMA_FLOP_PER_CYCLE = 256 * 4 * 1024.0  # dense f16: 256 CUs x 4 SIMDs x 32x32x16x2 FLOP per 32 cycles


def prefill_flop(pos0: int, tokens: int) -> float:
    """Causal-useful FLOP of one layer: n_head * sum_t (pos0+t+1) * 4 * head_dim."""
    pairs = tokens * pos0 + tokens * (tokens + 1) // 2
    return float(H * pairs * 4 * HD)


def decode_bytes(seq_total: int) -> float:
    """K+V cache bytes one layer's decode must read: 2 * n_kv * rows * 272."""
    return float(2 * KV * seq_total * ROW)


def measured_traffic(workload: str, kernels, largest=()):
    """HBM bytes per launch (read + written) of the named kernels, from the committed
    counter runs in profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled
    by a plain copy of known size); None when that file has no entry."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            t = json.load(f).get(workload, {})
    except OSError:
        return None
    total, seen = 0.0, False
    for name, v in t.items():
        if any(k in name for k in kernels):
            total += v["read_bytes"] + v["written_bytes"]
            seen = True
        elif any(k in name for k in largest):
            # a kernel that the run also launches at other sizes: its largest dispatch is the one meant
            total += v.get("max_read_bytes", v["read_bytes"]) + v.get("max_written_bytes", v["written_bytes"])
            seen = True
    return total if seen else None


class Timer:
    """HIP events on torch's current stream (the stream every launch below uses)."""

    def __init__(self, torch):
        self.torch = torch
        self.a = torch.cuda.Event(enable_timing=True)
        self.b = torch.cuda.Event(enable_timing=True)

    def __enter__(self):
        self.a.record()
        return self

    def __exit__(self, *exc):
        self.b.record()
        self.b.synchronize()
        self.ms = self.a.elapsed_time(self.b)


def timed(torch, fn, steps, warm=3, wall=False, min_ms=MIN_TIMED_MS):
    """Mean duration of fn(i) in ms over max(steps, what fills `min_ms`) calls, by HIP events on the launch
    stream (wall: by the host clock between two synchronisations); returns (ms per call, ms timed, calls)."""
    for i in range(warm):
        fn(i)
    probe = max(1, min(steps, 8))
    with Timer(torch) as t:
        for i in range(probe):
            fn(i)
    n = max(steps, int(1.1 * min_ms / max(t.ms / probe, 1e-4)) + 1)
    while True:
        if wall:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(n):
                fn(i)
            torch.cuda.synchronize()
            total = (time.perf_counter() - t0) * 1e3
        else:
            with Timer(torch) as t:
                for i in range(n):
                    fn(i)
            total = t.ms
        if total >= min_ms:
            break
        n = int(n * 1.2 * min_ms / max(total, 1e-3)) + 1  # (the short run was slower per call than the long one)
    return total / n, total, n


GRAPH_CAPTURE_FAILED = []  # messages of captures that failed (the figures concerned were then timed eagerly)


def timed_graph(torch, fn, calls, min_ms=MIN_TIMED_MS):
    """Mean duration of fn(i) in ms with fn(0) .. fn(calls - 1) captured once in a HIP graph and the graph
    replayed until `min_ms` of work have been timed (HIP events around the replays): what the launches cost when
    the host does not issue them one by one -- a call through Python and ctypes takes about 12 us of host time,
    more than a short launch runs.  Returns (ms per call, ms timed, calls timed)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(calls):
            fn(i)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(calls):
                fn(i)
    except Exception as e:  # (no box has refused a capture so far; if one does, say so and time the calls one by one)
        GRAPH_CAPTURE_FAILED.append(repr(e))
        torch.cuda.synchronize()
        return timed(torch, fn, calls, min_ms=min_ms)
    ms, total, n = timed(torch, lambda i: graph.replay(), 2, 2, min_ms=min_ms)
    return ms / calls, total, n * calls


def counters(workload: str, kernel: str):
    """Clock and MFMA-busy share of `kernel` in the committed counter run of `workload`
    (profiles/mfma_counters.json: rocprofv3 --pmc on this benchmark's --only legs), or {}."""
    try:
        with open(os.path.join(ROOT, "profiles", "mfma_counters.json")) as f:
            t = json.load(f).get(workload, {})
    except OSError:
        return {}
    for name, v in t.items():
        if kernel in name:
            if v.get("us", 0.0) < 500.0:
                # (GRBM_GUI_ACTIVE also counts the cycles around a dispatch: over a launch of tens of microseconds
                # the quotient is no clock, 2.8 "GHz" for the 25-us kernel)
                return {"mfma_busy": v.get("mfma_busy"),
                        "mfma_busy_source": "profiles/mfma_counters.json (SQ_VALU_MFMA_BUSY_CYCLES; a lower bound for a "
                                            "launch this short)"}
            return {"clock_ghz": v.get("clock_ghz"), "mfma_busy": v.get("mfma_busy"),
                    "clock_source": "profiles/mfma_counters.json (GRBM_GUI_ACTIVE / 8 / kernel duration)"}
    return {}


def mfma_yardstick(torch, attn, steps=4):
    """A loop of independent v_mfma_f32_32x32x16_f16 on one wave per SIMD of every CU: the rate the MFMA
    pipes reach with nothing else to do, and the clock the chip holds under that load."""
    wgs, iters = 256, 20000
    sink = torch.zeros(4, dtype=torch.float32, device="cuda")
    clocks = torch.zeros(2, dtype=torch.int64, device="cuda")
    ms, total, n = timed(torch, lambda i: attn.bench_mfma_f16(wgs, iters, sink, clocks), steps)
    flop = wgs * 4 * iters * 8 * 32768.0
    c = clocks.cpu().tolist()
    ghz = c[0] / max(c[1], 1) * 0.1
    tf = flop / (ms * 1e-3) / 1e12
    return {"workload": "256 workgroups x 4 waves (one per SIMD) x 20,000 x 8 independent v_mfma_f32_32x32x16_f16",
            "tflops": tf, "frac_of_peak": tf / MFMA_F16_PEAK_TF, "clock_ghz": ghz,
            "frac_at_that_clock": tf * 1e12 / (MFMA_FLOP_PER_CYCLE * ghz * 1e9),
            "ms_per_launch": ms, "timed_ms": total, "steps_timed": n}


def stream_yardstick(torch, attn, pairs, bytes_each, steps):
    """One launch per (k, v) pair that only reads bytes_each bytes of each, rotating over the pairs: GB/s of
    the better of the two load forms, with both times."""
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    bytes_each = bytes_each // 8704 * 8704
    res = {}
    for mode, name in ((0, "global_load_lds"), (1, "register_loads")):
        def one(i, mode=mode):
            k, v = pairs[i % len(pairs)]
            attn.bench_stream_read(k, v, bytes_each, mode, sink)
        ms, total, n = timed_graph(torch, one, 4 * len(pairs))
        res[name] = {"us_per_launch": ms * 1e3, "gbs": 2 * bytes_each / (ms * 1e-3) / 1e9, "timed_ms": total}
    best = max(res.values(), key=lambda r: r["gbs"])
    return {"achievable": best["gbs"], "bytes_per_launch": 2 * bytes_each, **{k: v for k, v in res.items()}}


def fill_cache_normal(torch, attn, k_cache, v_cache, stride, rows, gen, dtype=0):
    """Quantize N(0,1) rows into a [KV][stride][272] (q8_0) or [..][144] (q4_0, dtype 1) cache pair
    with the library's own append kernel, in slabs so the f32 source stays small."""
    slab = 8192
    for s0 in range(0, rows, slab):
        n = min(slab, rows - s0)
        kf = torch.randn((n, KV, HD), device="cuda", dtype=torch.float32, generator=gen)
        vf = torch.randn((n, KV, HD), device="cuda", dtype=torch.float32, generator=gen)
        attn.kv_encode_bulk(dtype, kf, vf, k_cache, v_cache, KV, HD, stride, s0, 0, n)
    torch.cuda.synchronize()


# ---------------------------------------------------------------------------------------
# prefill: rope + append + attention + gate
# ---------------------------------------------------------------------------------------

def bench_prefill(torch, attn, tokens, pos0, steps, warmup, layers, prefix_fill=True, mfma=None):
    stride = (pos0 + tokens + 63) // 64 * 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED0002 + pos0)
    caches = []
    for _ in range(layers):
        k = torch.zeros((KV, stride, ROW), dtype=torch.uint8, device="cuda")
        v = torch.zeros((KV, stride, ROW), dtype=torch.uint8, device="cuda")
        if pos0 > 0 and prefix_fill:
            fill_cache_normal(torch, attn, k, v, stride, pos0, gen)
        caches.append((k, v))
    # Every layer has its own activations as well (q, the chunk's K/V rows, gate, out: 75 MB per layer at
    # 672 tokens), so that a step finds none of its operands in the 256 MiB Infinity Cache from the
    # step before; the split scratch is one buffer, as it is in an engine.
    acts = []
    for _ in range(layers):
        acts.append((torch.randn((tokens, H, HD), device="cuda", generator=gen),
                     torch.randn((tokens, KV, HD), device="cuda", generator=gen),
                     torch.randn((tokens, KV, HD), device="cuda", generator=gen),
                     torch.randn((tokens, H, HD), device="cuda", generator=gen),
                     torch.empty((tokens, H, HD), device="cuda")))
    splits = attn.chunk_splits(pos0, tokens, KV)  # 0: the keys are cut inside the workgroups, no scratch
    slices = attn.chunk_slices(pos0, tokens, KV)  # the attention over the f16 copy is always the sliced kernel
    acc = ml = None
    if max(splits, slices) >= 2:
        acc, ml = attn.chunk_scratch(tokens, H, max(splits, slices))
    attn.rope_table(THETA, NROT, max(pos0 + tokens, 1024))
    # the f16 copy of every layer cache, current up to the prefix (as earlier chunks would have left it)
    copies = []
    for k, v in caches if splits != 0 else []:
        c = attn.kv_f16_alloc(stride, KV)
        if pos0 > 0:
            attn.kv_f16_rows(0, k, v, c, KV, HD, stride, 0, pos0)
        copies.append(c)

    def attention(i):
        k, v = caches[i % layers]
        q, kx, vx, gate, out = acts[i % layers]
        attn.chunk_attention_q8_split(q, k, v, out, H, KV, HD, pos0, tokens, 1, stride, acc, ml,
                                      splits)

    def attention_copy(i):
        q, kx, vx, gate, out = acts[i % layers]
        attn.chunk_attention_kv_f16(q, copies[i % layers], None, out, None, H, KV, HD, pos0, tokens, stride,
                                    acc, ml, slices)

    def step_copy(i, rebuild=False):
        # the same step with the attention reading the f16 copy of the cache: the chunk's rows are added
        # to the copy after the append (rebuild: the whole copy is made again from row 0, what a caller
        # does who keeps one copy for all layers)
        k, v = caches[i % layers]
        q, kx, vx, gate, out = acts[i % layers]
        attn.rope_encode_chunk(q, kx, vx, k, v, H, KV, HD, NROT, THETA, pos0, tokens, 0, stride)
        if rebuild:
            attn.kv_f16_rows(0, k, v, copies[i % layers], KV, HD, stride, 0, pos0 + tokens)
        else:
            attn.kv_f16_rows(0, k, v, copies[i % layers], KV, HD, stride, pos0, tokens)
        attn.chunk_attention_kv_f16(q, copies[i % layers], gate, out, None, H, KV, HD, pos0, tokens, stride,
                                    acc, ml, slices)

    def step(i):
        # RoPE and the append share one launch; the gate is applied where the attention result is
        # written (same bits as the separate kernels, two launches and one pass over the rows less)
        k, v = caches[i % layers]
        q, kx, vx, gate, out = acts[i % layers]
        if splits == 0:
            # the in-workgroup kernel rotates the query rows where it loads them: the first launch rotates and
            # appends the K/V rows only, and q is never rewritten (same bits in `out`)
            attn.rope_encode_chunk(None, kx, vx, k, v, H, KV, HD, NROT, THETA, pos0, tokens, 0, stride)
            attn.chunk_attention_rope_q8(q, k, v, gate, out, None, H, KV, HD, NROT, THETA, pos0, tokens, 1, stride,
                                         acc, ml, splits)
            return
        attn.rope_encode_chunk(q, kx, vx, k, v, H, KV, HD, NROT, THETA, pos0, tokens, 0, stride)
        attn.chunk_attention_q8_split_gate(q, k, v, gate, out, H, KV, HD, pos0, tokens, 1, stride,
                                           acc, ml, splits)

    def step_unfused(i):
        k, v = caches[i % layers]
        q, kx, vx, gate, out = acts[i % layers]
        attn.rope_chunk(q, kx, H, KV, HD, NROT, THETA, pos0, tokens)
        attn.kv_encode_bulk(0, kx, vx, k, v, KV, HD, stride, pos0, 0, tokens)
        attention(i)
        attn.q_gate(out, gate, out)

    unfused_ms, _, _ = timed(torch, step_unfused, steps, warmup, wall=True)
    wall_ms, wall_total, wall_n = timed(torch, step, steps, warmup, wall=True)
    # (a short step, issued call by call from Python, is partly the host's time: the same steps replayed from a
    # HIP graph, for comparison)
    graph_ms = timed_graph(torch, step, 2 * layers)[0] if wall_ms < 0.2 else None
    # the f16 copy of the cache serves long prefixes: the sliced kernel over it is not what a chunk near
    # position 0 would run (splits == 0), so that leg is left out there
    with_copy = splits != 0
    copy_ms = timed(torch, step_copy, steps, warmup, wall=True)[0] if with_copy else None
    copy_rebuilt_ms = timed(torch, lambda i: step_copy(i, True), steps, warmup, wall=True)[0] if with_copy else None

    # the attention launch alone, HIP events on the launch stream
    attn_ms, attn_total, attn_n = timed(torch, attention, steps, min(warmup, 3))
    attn_copy_ms = timed(torch, attention_copy, steps, min(warmup, 3))[0] if with_copy else None
    flop = prefill_flop(pos0, tokens)
    tf = flop / (attn_ms * 1e-3) / 1e12
    # A scratch sized for more slices than the sliced kernel would use: the call writes the live rows of the
    # cache as f16 tiles into the tail of the scratch and runs `slices` slices of the 64-token kernel over them.
    tiles_path = splits > slices >= 2
    # What an engine gets that keeps the reference's own scratch: 8 slices, allocated once
    # (crates/hipml-model/src/gpu/prefill.rs:159-166, gpu/attn_tile.rs:122-151): no room for the tiles, so the
    # call runs the kernel that dequantizes for itself.
    ref_scratch = None
    if tiles_path:
        ref_splits = 8

        def attention_ref(i):
            k, v = caches[i % layers]
            q, kx, vx, gate, out = acts[i % layers]
            attn.chunk_attention_q8_split(q, k, v, out, H, KV, HD, pos0, tokens, 1, stride, acc, ml, ref_splits)
        ref_ms, ref_total, _ = timed(torch, attention_ref, steps, min(warmup, 3))
        ref_scratch = {"note": "the same attention launch with the scratch an unchanged reference engine allocates "
                               "(8 slices): chunk_q8_kernel<split> + chunk_combine_kernel, no f16 tiles",
                       "splits": ref_splits, "attn_ms": ref_ms, "timed_ms": ref_total,
                       "frac": flop / (ref_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TF}
    # The same calls with every layer cache registered once (hipml_kv_f16_attach, what an engine does where it
    # allocates the cache): the library keeps the f16 tiles itself, the append converts the chunk's rows and the
    # attention through the reference's entry point reads them; no tiles are made per call.
    shadow = None
    if with_copy:
        for (k, v), c in zip(caches, copies):
            attn.kv_f16_attach(0, k, v, c, KV, HD, stride, pos0)
        try:
            sh_ms, sh_total, sh_n = timed(torch, step, steps, warmup, wall=True)
            sh_attn_ms, sh_attn_total, sh_attn_n = timed(torch, attention, steps, min(warmup, 3))
        finally:
            for k, v in caches:
                attn.kv_f16_detach(k)
        shadow = {"note": "every layer cache registered once with hipml_kv_f16_attach: rope + append (which converts "
                          "the chunk's rows) + hipml_attn_chunk_q8_split_gate reading the library-kept f16 tiles",
                  "ms_per_step": sh_ms, "tok_per_s": tokens / (sh_ms * 1e-3), "timed_ms": sh_total, "steps_timed": sh_n,
                  "attn_ms": sh_attn_ms, "attn_timed_ms": sh_attn_total,
                  "attn_frac": flop / (sh_attn_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TF,
                  "slices_run": min(max(splits, slices), slices)}
    rows_bytes = 2 * tokens * H * HD * 4 + 2 * KV * (pos0 + tokens) * ROW
    wl = {(672, 0): "prefill672", (2048, 100_000): "chunk100k"}.get((tokens, pos0), "")
    # (the attention-only launch timed here takes no gate and rotated query rows: <q4_0 false, in-kernel RoPE false>)
    if splits == 0:
        kernel, traffic = "chunk_wg_kernel", measured_traffic(wl, ["chunk_wg_kernel<false, false>"])
    elif tiles_path:
        kernel = "chunk_f16_t64_kernel"
        traffic = measured_traffic(wl, ["chunk_f16_t64_kernel", "chunk_combine_kernel"], ["kv_f16_tiles_kernel<false>"])
    else:
        kernel = "chunk_q8_kernel"
        traffic = measured_traffic(wl, ["chunk_q8_kernel<true, false, false>", "chunk_q8_kernel<false, false, false>",
                                        "chunk_combine_kernel"])
    res = {
        "workload": f"prefill {tokens}@{pos0}: rope + q8_0 append + causal GQA attention + gate, "
                    f"1 layer, {H}q/{KV}kv heads, head_dim {HD}",
        "tokens": tokens, "pos0": pos0, "splits": splits, "slices_over_f16_copy": slices, "layers_rotated": layers,
        "scratch_slices": max(splits, slices), "slices_run": slices if tiles_path else splits,
        "ms_per_step": wall_ms, "timed_ms": wall_total, "steps_timed": wall_n,
        "tok_per_s": tokens / (wall_ms * 1e-3),
        "ms_per_step_separate_launches": unfused_ms,
        "ms_per_step_graph_replay": graph_ms,
        "attn_ms": attn_ms,
        "attn_tok_per_s": tokens / (attn_ms * 1e-3),
        "reference_scratch_8_slices": ref_scratch,
        "attached_f16_shadow": shadow,
        "over_f16_copy": None if not with_copy else {
            "note": "the same step with the attention reading an f16 copy of the cache that the step keeps "
                    "current (hipml_kv_f16_rows for the chunk's rows after the append, then "
                    "hipml_attn_chunk_kv_f16); rebuilt = the whole copy made again from row 0 in every step",
            "ms_per_step": copy_ms, "tok_per_s": tokens / (copy_ms * 1e-3),
            "ms_per_step_copy_rebuilt": copy_rebuilt_ms,
            "attn_ms": attn_copy_ms, "attn_frac": flop / (attn_copy_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TF,
            "copy_bytes_per_layer": attn.kv_f16_bytes(stride, KV)},
        "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_F16_PEAK_TF, "unit": "TFLOP/s",
                     "frac": tf / MFMA_F16_PEAK_TF, "traffic": traffic,
                     "achievable": None if mfma is None else mfma["tflops"],
                     "frac_of_achievable": None if mfma is None else tf / mfma["tflops"],
                     **counters(wl, kernel),
                     "kernel": "chunk_wg_kernel" if splits == 0 else
                     "kv_f16_tiles_kernel + chunk_f16_t64_kernel + chunk_combine_kernel" if tiles_path else
                     "chunk_q8_kernel" + (" + chunk_combine_kernel" if splits >= 2 else ""),
                     "flop_per_launch": flop, "launch_ms": attn_ms, "timed_ms": attn_total, "steps_timed": attn_n,
                     # the same launch against the other roof: the f32 rows it has to move (Q in, rows out; the
                     # attention-only launch timed here takes no gate) and the cache rows once, over 8 TB/s
                     "algorithmic_bytes": rows_bytes,
                     "hbm_frac": rows_bytes / (attn_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
    }
    if tiles_path and shadow is not None:
        # Deep in a prefix the entry's figures are those of an engine that has registered its caches (the
        # integration this library documents); what the same calls cost without that is kept beside them.
        res["tiles_made_per_call_in_the_scratch"] = {
            "note": "no shadow registered, scratch sized by hipml_attn_chunk_splits: every call writes the live "
                    "rows as f16 tiles into the tail of the scratch first (kv_f16_tiles_kernel)",
            "ms_per_step": wall_ms, "attn_ms": attn_ms, "timed_ms": attn_total, "frac": tf / MFMA_F16_PEAK_TF,
            "traffic": traffic}
        tfs = flop / (shadow["attn_ms"] * 1e-3) / 1e12
        res.update({"ms_per_step": shadow["ms_per_step"], "timed_ms": shadow["timed_ms"],
                    "steps_timed": shadow["steps_timed"], "tok_per_s": shadow["tok_per_s"],
                    "attn_ms": shadow["attn_ms"], "attn_tok_per_s": tokens / (shadow["attn_ms"] * 1e-3)})
        res["workload"] += "; every layer cache registered once with hipml_kv_f16_attach"
        res["roofline"].update({
            "achieved": tfs, "frac": tfs / MFMA_F16_PEAK_TF,
            "frac_of_achievable": None if mfma is None else tfs / mfma["tflops"],
            "traffic": measured_traffic(wl, ["chunk_f16_t64_kernel", "chunk_combine_kernel"]),
            "kernel": "chunk_f16_t64_kernel + chunk_combine_kernel (f16 tiles kept by the library)",
            "launch_ms": shadow["attn_ms"], "timed_ms": shadow["attn_timed_ms"],
            "hbm_frac": rows_bytes / (shadow["attn_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS})
    return res


# ---------------------------------------------------------------------------------------
# decode
# ---------------------------------------------------------------------------------------

def bench_decode(torch, attn, seq, steps, warmup, layers, dtype=0, one_launch=False):
    row = ROW if dtype == 0 else 144
    stride = seq
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED0003 + seq)
    caches = []
    for _ in range(layers):
        k = torch.empty((KV, stride, row), dtype=torch.uint8, device="cuda")
        v = torch.empty((KV, stride, row), dtype=torch.uint8, device="cuda")
        fill_cache_normal(torch, attn, k, v, stride, seq, gen, dtype)
        caches.append((k, v))
    q = torch.randn((H, HD), device="cuda", generator=gen)
    out = torch.empty((H, HD), device="cuda")
    splits = attn.decode_splits(seq, KV)
    acc = torch.empty((H, splits, HD), device="cuda")
    ml = torch.empty((H, splits, 2), device="cuda")
    stepbuf = torch.tensor([seq - 1, seq, 0, 0, seq - 1, seq - 1, seq - 1, seq - 1],
                           dtype=torch.int32, device="cuda")

    def plain(i):
        k, v = caches[i % layers]
        attn.attn_decode_kv(stepbuf, dtype, q, k, v, acc, ml, out, H, KV, HD, stride, SCALE, splits)

    calls = steps * layers
    eager_us = timed(torch, plain, calls, warmup * layers)[0] * 1e3
    # The figures of this entry are replays of a HIP graph that holds 4 passes over the layer caches, as an
    # engine issues its decode step; issued call by call from Python the same launches are bound by the host at
    # short depths (us_per_layer_eager).
    in_graph = 4 * layers
    ms, total, n = timed_graph(torch, plain, in_graph)
    us = ms * 1e3
    # the same with the sigmoid output gate: in the merge kernel, and as the separate launch it replaces
    gate = torch.randn((H, HD), device="cuda", generator=gen)

    def gated(i):
        k, v = caches[i % layers]
        attn.attn_decode_kv_gate(stepbuf, dtype, q, k, v, acc, ml, out, gate, H, KV, HD, stride, SCALE, splits)

    def gate_apart(i):
        plain(i)
        attn.q_gate(out, gate, out, H * HD)

    tg = timed_graph(torch, gated, in_graph)[0] * 1e3
    ts = timed_graph(torch, gate_apart, in_graph)[0] * 1e3
    # the form whose workgroups merge the key splits themselves (one launch instead of two; q8_0 only)
    one_launch_us = None
    if one_launch and dtype == 0:
        before = attn.decode_one_launch(1)
        try:
            one_launch_us = timed_graph(torch, plain, in_graph)[0] * 1e3
        finally:
            attn.decode_one_launch(before)
    nbytes = decode_bytes(seq) * row // ROW
    gbs = nbytes / (us * 1e-6) / 1e9
    traffic = measured_traffic({(8192, 0): "decode8k", (32768, 0): "decode32k", (32768, 1): "decode32k_q4"}.get((seq, dtype), ""),
                               ["decode_q8_kernel", "decode_q4_kernel", "decode_reduce"])
    # what a launch that only reads the same bytes reaches on this box, same rotation over the layer caches
    ys = stream_yardstick(torch, attn, caches, KV * stride * row, steps)
    return {
        "workload": f"decode 1 query @ depth {seq}, {'q8_0' if dtype == 0 else 'q4_0'} cache, "
                    f"split-K {splits} + merge",
        "seq": seq, "splits": splits, "layers_rotated": layers,
        # (the scratch is sized for `splits`; one sequence runs at most one workgroup per CU over q8_0, and
        # over q4_0 below 24,576 rows)
        "splits_run": min(splits, max(256 // KV, 1)) if dtype == 0 or stride < 24576 else splits,
        "us_per_layer": us, "timed_ms": total, "steps_timed": n,
        "issued": f"HIP graph of {in_graph} calls, replayed", "us_per_layer_eager": eager_us,
        "us_per_layer_gate_fused": tg,
        "us_per_layer_gate_separate": ts,
        "us_per_layer_one_launch": one_launch_us,
        "pure_read": ys,
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS, "traffic": traffic,
                     "achievable": ys["achievable"], "frac_of_achievable": gbs / ys["achievable"],
                     "kernel": "decode_q8_kernel + decode_reduce128_kernel" if dtype == 0 else
                     "decode_q4_kernel + decode_reduce128_kernel",
                     "bytes_per_launch": nbytes, "launch_us": us, "timed_ms": total, "steps_timed": n},
    }


class Xorshift64Star:
    """The reference's generator (crates/hipml-core/src/rng.rs:19-38): state = seed | 1, xorshift
    12/25/27, multiply; uniform() = top 24 bits / 2^24.  Here for the seeded depths of the batch."""

    def __init__(self, seed: int):
        self.s = (seed | 1) & 0xFFFFFFFFFFFFFFFF

    def uniform(self) -> float:
        x = self.s
        x ^= x >> 12
        x ^= (x << 25) & 0xFFFFFFFFFFFFFFFF
        x ^= x >> 27
        self.s = x
        return (((x * 0x2545F4914F6CDD1D) & 0xFFFFFFFFFFFFFFFF) >> 40) / float(1 << 24)


def batch_case(slots=16, verify=4, lo=512, hi=16384):
    r = Xorshift64Star(0x5EED0005)
    depths = [lo + int(r.uniform() * (hi - lo + 1)) for _ in range(slots)]
    cols = [3 if s < verify else 1 for s in range(slots)]
    return depths, cols


def bench_batch(torch, attn, steps, warmup, layers):
    depths, cols = batch_case()
    slots = len(depths)
    stride = 16448
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED0005)
    slot_bytes = KV * stride * ROW
    caches = []
    for _ in range(layers):
        k = torch.zeros((slots, KV, stride, ROW), dtype=torch.uint8, device="cuda")
        v = torch.zeros((slots, KV, stride, ROW), dtype=torch.uint8, device="cuda")
        for s in range(slots):
            fill_cache_normal(torch, attn, k[s], v[s], stride, depths[s] + cols[s], gen)
        caches.append((k, v))
    rows = sum(cols)
    pos = []
    for s in range(slots):
        for c in range(cols[s]):
            pos += [depths[s] + c, depths[s] + c + 1]
    pos_d = torch.tensor(pos, dtype=torch.int32, device="cuda")
    q = torch.randn((rows, H, HD), device="cuda", generator=gen)
    out = torch.empty((rows, H, HD), device="cuda")
    splits = attn.batch_splits(stride, KV, slots)
    acc = torch.empty((rows, H, splits, HD), device="cuda")
    ml = torch.empty((rows, H, splits, 2), device="cuda")

    def one(i):
        k, v = caches[i % layers]
        attn.attn_decode_batch_cols(0, pos_d, q, k, v, acc, ml, out, H, KV, HD, stride, SCALE,
                                    splits, slot_bytes, H * splits * HD, H * splits * 2, H * HD,
                                    cols)

    ms, total, n = timed(torch, one, steps * layers, warmup * layers)
    us = ms * 1e3
    live = sum(d + c for d, c in zip(depths, cols))
    nbytes = decode_bytes(live)
    gbs = nbytes / (us * 1e-6) / 1e9
    traffic = measured_traffic("batch16", ["decode_q8_kernel", "decode_reduce"])
    # the pure read of as many bytes (the first half of them from each of a layer's two arrays)
    flat = [(k.reshape(-1), v.reshape(-1)) for k, v in caches]
    ys = stream_yardstick(torch, attn, flat, int(nbytes) // 2, steps)
    return {
        "workload": f"batched decode, {slots} slots, depths U[512,16384] (seeded), "
                    f"slots 0..3 carry 3 query rows (MTP verify), one launch",
        "slots": slots, "rows": rows, "live_rows": live, "splits": splits, "layers_rotated": layers,
        "us_per_layer": us, "timed_ms": total, "steps_timed": n,
        "pure_read": ys,
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS, "traffic": traffic,
                     "achievable": ys["achievable"], "frac_of_achievable": gbs / ys["achievable"],
                     "kernel": "decode_q8_kernel + decode_reduce128_kernel",
                     "bytes_per_launch": nbytes, "launch_us": us, "timed_ms": total, "steps_timed": n},
    }


def bench_batch_layer(torch, attn, steps, layers):
    """One plain step of the batched engine through the attention block: 16 sequences at the seeded
    depths of the batched benchmark, one row each -- front end with append (per-row positions,
    per-slot caches), batched attention with the gate in the merge, W_o over the 16 rows: 4 launches."""
    depths, _ = batch_case()
    slots, stride = len(depths), 16448
    m, k = 5120, H * HD
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED000B)
    kvs, ws = [], []
    for _ in range(layers):
        kv = attn.BatchKv(slots, H, KV, HD, stride)
        for s in range(slots):
            fill_cache_normal(torch, attn, kv.k[s], kv.v[s], stride, depths[s], gen)
        kvs.append(kv)
        ws.append(random_q8_0_weights(torch, m, k, gen))
    pos = torch.tensor([[d, d + 1] for d in depths], dtype=torch.int32, device="cuda")
    qg = torch.randn((slots, H, 2 * HD), device="cuda", generator=gen)
    kx = torch.randn((slots, KV, HD), device="cuda", generator=gen)
    vx = torch.randn((slots, KV, HD), device="cuda", generator=gen)
    qw = torch.ones(HD, device="cuda")
    kw = torch.ones(HD, device="cuda")
    q = torch.empty((slots, H, HD), device="cuda")
    gate = torch.empty((slots, H, HD), device="cuda")
    out = torch.empty((slots, H, HD), device="cuda")
    y = torch.empty((slots, m), device="cuda")
    attn.rope_table(THETA, NROT, stride + 64)

    def one(i):
        kv, w = kvs[i % layers], ws[i % layers]
        kv.front_append(qg, kx, vx, q, gate, qw, kw, NROT, THETA, 1e-6, pos)
        kv.decode(pos, q, out, SCALE, gate=gate)
        attn.gemv_q8_0_rows(w, out, y, m, k, slots)

    ms, total, n = timed(torch, one, steps * layers, 3 * layers)
    return {"workload": f"batched step, {slots} sequences at depths U[512,16384] (seeded), one row each: front "
                        f"end with append + attention with gate + W_o, {layers} layers rotated (4 launches "
                        f"per layer)",
            "us_per_layer": ms * 1e3, "timed_ms": total, "steps_timed": n, "live_rows": sum(depths) + slots}


def bench_front(torch, attn, tokens, steps):
    """Attention front end over a chunk: q|gate split + head RMS norm + RoPE (one launch)."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED0006)
    qg = torch.randn((tokens, H, 2 * HD), device="cuda", generator=gen)
    k0 = torch.randn((tokens, KV, HD), device="cuda", generator=gen)
    k = k0.clone()
    qw = torch.ones(HD, device="cuda")
    kw = torch.ones(HD, device="cuda")
    q = torch.empty((tokens, H, HD), device="cuda")
    gate = torch.empty((tokens, H, HD), device="cuda")
    attn.rope_table(THETA, NROT, max(tokens, 1024))
    ms, total, n = timed(torch, lambda i: attn.chunk_front(qg, k, q, gate, qw, kw, H, KV, HD, NROT, THETA, 1e-6, 0,
                                                            tokens), steps)
    us = ms * 1e3
    nbytes = tokens * (H * 2 * HD + 2 * H * HD + 2 * KV * HD) * 4  # qg read, q + gate written, k both
    gbs = nbytes / (us * 1e-6) / 1e9
    return {"workload": f"attention front end, {tokens} rows: q|gate split + head RMS norm + RoPE",
            "us": us, "bytes": nbytes, "timed_ms": total, "steps_timed": n,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": gbs / HBM_PEAK_GBS, "traffic": None, "kernel": "front_kernel"}}


def bench_decode_layer(torch, attn, seq, steps, layers):
    """One decode token through the attention block of `layers` layers: front end (q|gate split, head
    norms, RoPE), append, split-K attention with the gate in the merge, output projection -- issued
    eagerly, and captured once in a HIP graph and replayed (positions live in the device step buffer)."""
    m, k = 5120, H * HD
    stride = seq + 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED0009)
    caches, ws = [], []
    for _ in range(layers):
        kc = torch.empty((KV, stride, ROW), dtype=torch.uint8, device="cuda")
        vc = torch.empty((KV, stride, ROW), dtype=torch.uint8, device="cuda")
        fill_cache_normal(torch, attn, kc, vc, stride, seq, gen)
        caches.append((kc, vc))
        ws.append(random_q8_0_weights(torch, m, k, gen))
    qg = torch.randn((H, 2 * HD), device="cuda", generator=gen)
    kx0 = torch.randn((KV, HD), device="cuda", generator=gen)
    kx = kx0.clone()
    vx = torch.randn((KV, HD), device="cuda", generator=gen)
    qw = torch.ones(HD, device="cuda")
    kw = torch.ones(HD, device="cuda")
    q = torch.empty((H, HD), device="cuda")
    gate = torch.empty((H, HD), device="cuda")
    out = torch.empty((H, HD), device="cuda")
    y = torch.empty((1, m), device="cuda")
    splits = attn.decode_splits(stride, KV)
    acc = torch.empty((H, splits, HD), device="cuda")
    ml = torch.empty((H, splits, 2), device="cuda")
    step = torch.tensor([seq, seq + 1, 0, 0, seq, seq, seq, seq], dtype=torch.int32, device="cuda")
    attn.rope_table(THETA, NROT, stride + 64)

    def one_pass(fused=True):
        for (kc, vc), w in zip(caches, ws):
            if fused:
                attn.attn_front_encode(step, 0, qg, q, gate, kx, vx, qw, kw, kc, vc, H, KV, HD, NROT,
                                       (11, 11, 10, 0), THETA, 1e-6, stride)
            else:
                attn.attn_front(qg, q, gate, kx, qw, kw, H, KV, HD, NROT, (11, 11, 10, 0), step[4:], THETA, 1e-6)
                attn.kv_encode(step, 0, kx, vx, kc, vc, KV, HD, stride)
            attn.attn_decode_kv_gate(step, 0, q, kc, vc, acc, ml, out, gate, H, KV, HD, stride, SCALE, splits)
            attn.gemv_q8_0_rows(w, out, y, m, k, 1)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        one_pass()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        one_pass()
    for _ in range(3):
        one_pass()
        one_pass(False)
        graph.replay()
    te, total, n = timed(torch, lambda i: one_pass(), steps, 0)
    ts = timed(torch, lambda i: one_pass(False), steps, 0)[0]
    tg = timed(torch, lambda i: graph.replay(), steps, 0)[0]
    return {"workload": f"decode token @ depth {seq}: front end with append + attention with gate + W_o, "
                        f"{layers} layers per pass (4 launches per layer)",
            "us_per_layer_eager": te * 1e3 / layers, "timed_ms": total, "steps_timed": n * layers,
            "us_per_layer_graph_replay": tg * 1e3 / layers,
            "us_per_layer_eager_front_and_append_apart": ts * 1e3 / layers}


def bench_chunk_layer(torch, attn, tokens, pos0, steps, layers):
    """A chunk through the attention block: front end (q|gate split, head norms, RoPE) with the append,
    gated attention delivering f16 rows, W_o GEMM over them -- 4 launches -- beside the same work as
    the separate calls (front end, append, attention with gate, gate/convert pass, GEMM)."""
    m, k = 5120, H * HD
    stride = (pos0 + tokens + 63) // 64 * 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED000A)
    caches, ws = [], []
    for _ in range(layers):
        kc = torch.zeros((KV, stride, ROW), dtype=torch.uint8, device="cuda")
        vc = torch.zeros((KV, stride, ROW), dtype=torch.uint8, device="cuda")
        if pos0 > 0:
            fill_cache_normal(torch, attn, kc, vc, stride, pos0, gen)
        caches.append((kc, vc))
        ws.append(random_q8_0_weights(torch, m, k, gen))
    qg = torch.randn((tokens, H, 2 * HD), device="cuda", generator=gen)
    kx = torch.randn((tokens, KV, HD), device="cuda", generator=gen)
    vx = torch.randn((tokens, KV, HD), device="cuda", generator=gen)
    qw = torch.ones(HD, device="cuda")
    kw = torch.ones(HD, device="cuda")
    q = torch.empty((tokens, H, HD), device="cuda")
    gate = torch.empty((tokens, H, HD), device="cuda")
    out = torch.empty((tokens, H, HD), device="cuda")
    out16 = torch.empty((tokens, H, HD), dtype=torch.float16, device="cuda")
    y = torch.empty((tokens, m), device="cuda")
    splits = attn.chunk_splits(pos0, tokens, KV)
    acc = ml = None
    if splits >= 2:
        acc, ml = attn.chunk_scratch(tokens, H, splits)
    attn.rope_table(THETA, NROT, max(pos0 + tokens, 1024))

    def fused(i):
        (kc, vc), w = caches[i % layers], ws[i % layers]
        attn.chunk_front_encode(0, qg, kx, vx, q, gate, qw, kw, kc, vc, H, KV, HD, NROT, THETA, 1e-6,
                                pos0, tokens, stride)
        attn.chunk_attention_q8_split_gate_f16(q, kc, vc, gate, out, out16, H, KV, HD, pos0, tokens, 1,
                                               stride, acc, ml, splits)
        attn.output_chunk_q8_0(w, None, None, y, m, k, tokens, out16)

    def apart(i):
        (kc, vc), w = caches[i % layers], ws[i % layers]
        attn.chunk_front(qg, kx, q, gate, qw, kw, H, KV, HD, NROT, THETA, 1e-6, pos0, tokens)
        attn.kv_encode_bulk(0, kx, vx, kc, vc, KV, HD, stride, pos0, 0, tokens)
        attn.chunk_attention_q8_split_gate(q, kc, vc, gate, out, H, KV, HD, pos0, tokens, 1, stride,
                                           acc, ml, splits)
        attn.output_chunk_q8_0(w, out, None, y, m, k, tokens, out16)

    res = {}
    for name, fn in (("us_per_layer", fused), ("us_per_layer_separate_calls", apart)):
        ms, total, n = timed(torch, fn, steps)
        res[name] = ms * 1e3
        if name == "us_per_layer":
            res["timed_ms"], res["steps_timed"] = total, n
    return {"workload": f"chunk {tokens}@{pos0} through front end with append + gated attention (f16 rows) "
                        f"+ W_o GEMM, {layers} layers rotated (4 launches per layer)", **res,
            "tok_per_s": tokens / (res["us_per_layer"] * 1e-6)}


def random_q8_0_weights(torch, m, k, gen):
    """[m][k/32] Q8_0 blocks with random payloads and the reference's case scale 2^-10 (f16 0x1400)."""
    w = torch.randint(0, 256, (m * (k // 32), 34), dtype=torch.uint8, device="cuda", generator=gen)
    w[:, 0] = 0x00
    w[:, 1] = 0x14
    return w.reshape(-1)


def bench_gemv(torch, attn, rows, steps, layers, m=5120, k=6144):
    """Output projection W_o (Q8_0, 6144 -> 5120) over `rows` activation rows, rotating over
    `layers` distinct matrices (33.4 MB each) so the weights come from HBM."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED0007)
    ws = [random_q8_0_weights(torch, m, k, gen) for _ in range(layers)]
    x = torch.randn((rows, k), device="cuda", generator=gen) * 0.5
    y = torch.empty((rows, m), device="cuda")
    one = lambda i: attn.gemv_q8_0_rows(ws[i % layers], x, y, m, k, rows)
    eager_us = timed(torch, one, steps * layers, layers)[0] * 1e3
    ms, total, n = timed_graph(torch, one, 4 * layers)  # (issued one by one from Python the launch is host-bound)
    us = ms * 1e3
    # algorithmic bytes: the weights once, however many passes the kernel makes over them
    nbytes = m * (k // 32) * 34
    gbs = nbytes / (us * 1e-6) / 1e9
    return {"workload": f"W_o projection, Q8_0 {m}x{k}, {rows} activation rows",
            "us_per_layer": us, "timed_ms": total, "steps_timed": n, "weight_bytes": m * (k // 32) * 34,
            "issued": f"HIP graph of {4 * layers} calls, replayed", "us_per_layer_eager": eager_us,
            "layers_rotated": layers,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": gbs / HBM_PEAK_GBS,
                         "traffic": measured_traffic({1: "gemv1", 24: "gemv24"}.get(rows, ""),
                                                     ["gemv_q8_dma_kernel", "gemv_q8_dma_tile_kernel", "gemv_q8_rows_kernel",
                                                      "gemv_q8_tile_kernel"]),
                         "kernel": ("gemv_q8_dma_kernel" if rows <= 8 else
                                    "gemv_q8_dma_tile_kernel" if rows >= 10 else "gemv_q8_tile_kernel"),
                         "bytes_per_launch": nbytes, "launch_us": us}}


def bench_gemm(torch, attn, tokens, steps, layers, m=5120, k=6144, mfma=None):
    """Output side of a prefill chunk: y = W_o (out * sigmoid(gate)), [tokens][6144] x W_o^T (Q8_0) on
    MFMA with f16 operands."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0x5EED0008)
    ws = [random_q8_0_weights(torch, m, k, gen) for _ in range(layers)]
    x = torch.randn((tokens, k), device="cuda", generator=gen) * 0.5
    y = torch.empty((tokens, m), device="cuda")
    gate = torch.randn((tokens, k), device="cuda", generator=gen)
    x16 = torch.empty((tokens, k), dtype=torch.float16, device="cuda")
    t32 = timed(torch, lambda i: attn.gemm_q8_0_f16(ws[i % layers], x, y, m, k, tokens), steps * layers, layers)[0]
    # the whole output side: gate + rounding to f16 in one pass, then the GEMM over f16 rows
    ms, total, n = timed(torch, lambda i: attn.output_chunk_q8_0(ws[i % layers], x, gate, y, m, k, tokens, x16),
                         steps * layers, layers)
    us = ms * 1e3
    flop = 2.0 * tokens * m * k
    tf = flop / (us * 1e-6) / 1e12
    wl = "gemm672" if tokens == 672 else ""
    return {"workload": f"W_o projection of a chunk, Q8_0 {m}x{k}, {tokens} tokens",
            "us_per_layer": us, "timed_ms": total, "steps_timed": n, "us_per_layer_f32_rows_no_gate": t32 * 1e3,
            "flop": flop, "layers_rotated": layers,
            "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_F16_PEAK_TF, "unit": "TFLOP/s",
                         "frac": tf / MFMA_F16_PEAK_TF,
                         "achievable": None if mfma is None else mfma["tflops"],
                         "frac_of_achievable": None if mfma is None else tf / mfma["tflops"],
                         **counters(wl, "gemm_q8_f16_kernel<true"),
                         "traffic": measured_traffic(wl, ["gate_f16_kernel", "gemm_q8_f16_kernel<true"]),
                         "kernel": "gate_f16_kernel + gemm_q8_f16_kernel",
                         "flop_per_launch": flop, "launch_us": us}}


def bench_copycal(torch, steps):
    """Plain device copy of a known size: the yardstick the HBM traffic counters
    (FETCH_SIZE / WRITE_SIZE) are scaled by."""
    n = 64 << 20
    a = torch.empty(n, dtype=torch.uint8, device="cuda")
    b = torch.ones(n, dtype=torch.uint8, device="cuda")
    ms, total, cnt = timed(torch, lambda i: a.copy_(b), steps)
    return {"workload": "device copy", "bytes_read": n, "bytes_written": n,
            "us_per_copy": ms * 1e3, "timed_ms": total, "steps_timed": cnt}


# ---------------------------------------------------------------------------------------
# CPU baseline (the oracle, timed; never part of the measured GPU path)
# ---------------------------------------------------------------------------------------

def cpu_prefill(orc, np, tokens, pos0, rows_sample=None, n_threads=1, budget=10.0):
    """The oracle on the headline workload, repeated for about `budget` seconds; the attention runs on
    `n_threads` threads over query heads (1 = the reference's own single-threaded path); returns
    (tok/s, seconds, repetitions)."""
    r = orc.Rng(0x5EED0002)
    stride = pos0 + tokens
    q = r.normal_array((tokens, H, HD))
    k = r.normal_array((stride, KV, HD))
    v = r.normal_array((stride, KV, HD))
    gate = r.normal_array((tokens, H, HD))
    sec = (11, 11, 10, 0)
    rows = None if rows_sample is None else np.asarray(rows_sample, dtype=np.int32)
    n = tokens if rows is None else len(rows)
    # the whole workload, repeated until about ten seconds of CPU work have been timed
    reps, total = 0, 0.0
    while total < budget and reps < 50:
        qq, kk = q.copy(), k.copy()
        t0 = time.perf_counter()
        for t in range(tokens):
            p = pos0 + t
            qq[t] = orc.rope_multi(qq[t], H, HD, NROT, sec, (p, p, p, p), THETA).reshape(H, HD)
            kk[p] = orc.rope_multi(kk[p], KV, HD, NROT, sec, (p, p, p, p), THETA).reshape(KV, HD)
        kb = orc.quantize(0, kk.transpose(1, 0, 2)).reshape(KV, stride, ROW)
        vb = orc.quantize(0, v.transpose(1, 0, 2)).reshape(KV, stride, ROW)
        o = orc.attn_chunk_kv(qq, kb, vb, H, KV, HD, pos0, tokens, stride, SCALE, rows=rows, n_threads=n_threads)
        orc.q_gate(o.ravel(), gate[:n].ravel())
        total += time.perf_counter() - t0
        reps += 1
    return n * reps / total, total, reps


def cpu_decode(orc, seq):
    r = orc.Rng(0x5EED0003 + seq)
    q = r.normal_array((H, HD))
    kb = orc.synthetic_blocks(0, KV * seq * 8, 11).reshape(KV, seq, ROW)
    vb = orc.synthetic_blocks(0, KV * seq * 8, 12).reshape(KV, seq, ROW)
    t0 = time.perf_counter()
    orc.attn_decode_kv(q, kb, vb, H, KV, HD, seq, SCALE)
    return (time.perf_counter() - t0) * 1e6


# ---------------------------------------------------------------------------------------

def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200,
                    help="steps of the headline workload to time at least (more are timed until 200 ms are full)")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--main-only", action="store_true", help="skip the 'also' workloads")
    ap.add_argument("--only", default="", help="run one workload alone (prefill672, decode8k, "
                    "decode32k, decode32k_one_launch, decode128k, chunk100k, batch16, mfma, front672, decode32k_q4, gemv1, gemv4, gemv16, gemm672, gemm2048, layer32k, layer672, blayer16, copycal) for profiling; prints its object")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the attention path needs no exchange "
              "between GPUs); run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch
    from hipml_amd import attn

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    attn.init(0)
    K, W = args.steps, args.warmup

    # (--steps is a lower bound on what every figure is averaged over; figures that would be timed for less
    # than MIN_TIMED_MS at that count repeat until they have been)
    if args.only:
        mf = lambda: mfma_yardstick(torch, attn)
        fn = {
            "prefill672": lambda: bench_prefill(torch, attn, 672, 0, K, W, LAYERS, mfma=mf()),
            "decode8k": lambda: bench_decode(torch, attn, 8192, K, W, LAYERS),
            "decode32k": lambda: bench_decode(torch, attn, 32768, K, W, LAYERS),
            "decode32k_one_launch": lambda: bench_decode(torch, attn, 32768, K, W, LAYERS, one_launch=True),
            "decode128k": lambda: bench_decode(torch, attn, 131072, K, W, LAYERS),
            "chunk100k": lambda: bench_prefill(torch, attn, 2048, 100_000, K, W, 2, mfma=mf()),
            "batch16": lambda: bench_batch(torch, attn, K, W, 4),
            "copycal": lambda: bench_copycal(torch, K),
            "mfma": mf,
            "front672": lambda: bench_front(torch, attn, 672, K),
            "decode32k_q4": lambda: bench_decode(torch, attn, 32768, K, 3, LAYERS, 1),
            "gemv1": lambda: bench_gemv(torch, attn, 1, K, LAYERS),
            "gemv4": lambda: bench_gemv(torch, attn, 4, K, LAYERS),
            "gemv16": lambda: bench_gemv(torch, attn, 16, K, LAYERS),
            "gemv24": lambda: bench_gemv(torch, attn, 24, K, LAYERS),
            "gemv64": lambda: bench_gemv(torch, attn, 64, K, LAYERS),
            "gemv128": lambda: bench_gemv(torch, attn, 128, K, LAYERS),
            "gemm24": lambda: bench_gemm(torch, attn, 24, K, LAYERS),
            "gemm128": lambda: bench_gemm(torch, attn, 128, K, LAYERS),
            "layer32k": lambda: bench_decode_layer(torch, attn, 32768, K, LAYERS),
            "blayer16": lambda: bench_batch_layer(torch, attn, K, 4),
            "layer672": lambda: bench_chunk_layer(torch, attn, 672, 0, K, 4),
            "gemm672": lambda: bench_gemm(torch, attn, 672, K, 4, mfma=mf()),
            "gemm2048": lambda: bench_gemm(torch, attn, 2048, K, 4, mfma=mf()),
        }[args.only]
        print(json.dumps(fn()))
        return 0

    mfma = mfma_yardstick(torch, attn)
    main_r = bench_prefill(torch, attn, 672, 0, K, W, LAYERS, mfma=mfma)
    line = {
        "metric": "prefill_attn_tok_per_s",
        "value": main_r["tok_per_s"],
        "unit": "tok/s",
        "n_gpus": 1, "steps": K, "warmup": W,
        "steps_timed": main_r["steps_timed"], "timed_ms": main_r["timed_ms"],
        "ms_per_step": main_r["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "dtype_note": "f16 MFMA operands (Q, dequantized q8_0 K/V, P), f32 accumulation and softmax",
        "data": "synthetic",
        "config": {"workload": main_r["workload"], "tokens": 672, "pos0": 0,
                   "layers_rotated": LAYERS, "splits": main_r["splits"]},
        "attn_only_tok_per_s": main_r["attn_tok_per_s"],
        "roofline": main_r["roofline"],
    }

    if not args.main_only:
        also = {}
        d_steps = 1  # passes over the 16 layer caches: the 200 ms rule sets the count
        also["mfma_32x32x16_f16"] = mfma
        also["decode_8192"] = bench_decode(torch, attn, 8192, d_steps, 2, LAYERS)
        torch.cuda.empty_cache()
        also["decode_32768"] = bench_decode(torch, attn, 32768, d_steps, 2, LAYERS, one_launch=True)
        torch.cuda.empty_cache()
        # beyond the two benchmark depths: shows what the same kernel does once launch and ramp-up
        # stop dominating (285 MB per layer)
        also["decode_131072"] = bench_decode(torch, attn, 131072, d_steps, 2, LAYERS)
        torch.cuda.empty_cache()
        also["chunk_2048_at_100000"] = bench_prefill(torch, attn, 2048, 100_000, 10, 2, 2, mfma=mfma)
        torch.cuda.empty_cache()
        also["front_672"] = bench_front(torch, attn, 672, 20)
        also["decode_32768_q4_0"] = bench_decode(torch, attn, 32768, d_steps, 2, LAYERS, 1)
        also["batch16_mtp"] = bench_batch(torch, attn, d_steps, 2, 4)
        torch.cuda.empty_cache()
        # the step after the path: output projection over Q8_0 weights (decode rows, then a chunk)
        also["wo_rows_1"] = bench_gemv(torch, attn, 1, d_steps, LAYERS)
        also["wo_rows_4"] = bench_gemv(torch, attn, 4, d_steps, LAYERS)
        also["wo_rows_24"] = bench_gemv(torch, attn, 24, d_steps, LAYERS)  # the batch of 16 slots with 4 verify groups
        torch.cuda.empty_cache()
        also["wo_chunk_672"] = bench_gemm(torch, attn, 672, 10, 4, mfma=mfma)
        torch.cuda.empty_cache()
        also["decode_layer_32768"] = bench_decode_layer(torch, attn, 32768, d_steps, LAYERS)
        torch.cuda.empty_cache()
        also["chunk_layer_672"] = bench_chunk_layer(torch, attn, 672, 0, 10, 4)
        torch.cuda.empty_cache()
        also["batch_layer_16"] = bench_batch_layer(torch, attn, d_steps, 4)
        torch.cuda.empty_cache()
        line["also"] = also

    if not args.no_cpu:
        from oracle import binding as orc
        tokps, secs, reps = cpu_prefill(orc, np, 672, 0)
        line["cpu_baseline"] = {
            "value": tokps, "unit": "tok/s", "cores": 1, "kind": "port",
            "sample": f"the whole headline workload {reps} times (672 tokens @ 0: rope + quantize + "
                      f"causal attention over the dequantized cache + gate), {secs:.1f} s in all, "
                      f"1 thread, scalar C restatement of the reference's CPU path",
            "host_cpus": os.cpu_count(),
        }
        # beside it: the same restatement with its attention spread over the box's CPU share
        nt = min(16, os.cpu_count() or 1)
        if nt > 1:
            mt, msecs, mreps = cpu_prefill(orc, np, 672, 0, n_threads=nt, budget=3.0)
            line["cpu_baseline"]["threads"] = {"value": mt, "unit": "tok/s", "cores": nt,
                                               "sample": f"the same workload {mreps} times, {msecs:.1f} s"}
        if not args.main_only:
            line["cpu_baseline"]["decode_us_per_layer"] = {
                "8192": cpu_decode(orc, 8192), "32768": cpu_decode(orc, 32768)}
    if GRAPH_CAPTURE_FAILED:
        line["graph_capture_failed"] = GRAPH_CAPTURE_FAILED
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

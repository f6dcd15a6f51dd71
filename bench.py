#!/usr/bin/env python3
"""Benchmark of the KV-cache / attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

A step is one pass of the hot path over one batch of synthetic input:

  decode workloads   one decode step = for every layer (append one token if the workload says so,
                     then split-K decode attention + merge).  Metric: KV bytes read per second.
  prefill workload   for every layer: append the 512-token chunk, then causal batched attention.
                     Metric: TFLOP/s.

The default workload is the one the headline metric is quoted on: 32 layers, FP8 KV, 32768 keys,
32/8/128 heads.  Inputs are resident in HBM before the timed region.  After the timed region the
same launches are replayed with HIP events around each launch of the dominant kernel (on the
stream it runs on) to obtain its average duration for the roofline entry, and the CPU oracle is
timed on a bounded sample of the same workload on the host cores of this machine.
Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0
MFMA_F32_PEAK_TFLOPS = 157.3      # dense f32 matrix rate: what an F32 cache is multiplied at


# HBM bytes per launch of the dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE
# (two runs) and scaled by what the same counters read for a plain 64 MiB device copy
# (FETCH_SIZE x 1.9991, WRITE_SIZE x 1.0 to KiB).  Only the workloads that were profiled have an entry.  Counters cannot
# be read from inside this process, so an entry names the summary it comes from and the digest of the kernel sources
# it was taken with: when the sources have changed since, the line reports null instead of a stale figure.
PROFILED_TRAFFIC = {
    "decode_fp8_32k_32layers": {
        "bytes": (65690 + 520) * 1024, "profile": "profiles/decode_fp8_32k_split_mfma_il_kernel.md",
        "sources": ('attn_decode.hip', 'attn_decode_il.h', 'rope_device.h', 'device_utils.h'), "sha256_16": "20976d6933688778"},
    "prefill_fp8_512x4608_32layers": {
        "bytes": (19411 + 10240) * 1024, "profile": "profiles/prefill_fp8_512x4608_batch_dma_kernel.md",
        "sources": ('attn_prefill.hip', 'attn_prefill_dma.h', 'device_utils.h'), "sha256_16": "01810eb838265063"},
}


def prefill_kernel_name(kv_label, head_dim, group):
    """The kernel attn_prefill.hip launches for a shape with 16-byte aligned buffers."""
    if kv_label == "FP32":
        return "batch_mfma_f32_kernel"
    if kv_label == "FP8" and head_dim == 128 and group >= 2:
        return "batch_dma_kernel"       # two heads per wavefront over FP8 rows: V loaded straight into LDS
    return "batch_mfma2_kernel"


def kernel_sources_digest(names):
    import hashlib
    h = hashlib.sha256()
    for n in names:
        with open(os.path.join(ROOT, "vulkanforge_amd", "csrc", n), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic(workload):
    """(bytes or None, where the figure comes from) for the roofline entry of `workload`."""
    e = PROFILED_TRAFFIC.get(workload)
    if e is None:
        return None, None
    if kernel_sources_digest(e["sources"]) != e["sha256_16"]:
        return None, e["profile"] + " (kernel sources changed since that profile: not reported)"
    return e["bytes"], e["profile"]


def host_cpu():
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"cpu_model": model, "hardware_concurrency": os.cpu_count()}


MFMA_DTYPE = "f16 mfma on value + remainder operand pairs, f32 accumulate"   # what the matrix-core kernels compute in


def mfma_decode_worker(dtype_label, head_dim):
    """Mirrors the library's choice: FP8 / F16 caches at head_dim 64 / 128 / 256 / 512 run on the matrix-core worker, and so
    do the multiples of 16 between 64 and 256 (on the next wider worker, tail masked off)."""
    return (os.environ.get("VFKV_DECODE_WORKER", "m")[:1] != "v" and dtype_label in ("FP8", "FP16")
            and (head_dim in (64, 128, 256, 512) or (64 < head_dim < 256 and head_dim % 16 == 0)))


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="decode_fp8_32k_32layers")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--f32-queries", action="store_true",
                    help="leave the queries as general f32 values instead of casting them to fp16 first")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch every kernel from Python instead of replaying one captured HIP graph per step")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="headline run only: skip the short runs of the other benchmark configurations ('workloads' array)")
    return ap.parse_args()


def fill_cache(torch, vf, fwd, wl, n_tokens, seed, outliers):
    """Seeded synthetic K/V: N(0,1) rounded to fp16 (or N(0,1)*0.5 with a 1 % tail at +-40), written
    through the append kernels so the cache holds exactly what the product would have written."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    cache = fwd.kv_cache
    chunk = 4096
    for layer in range(wl.n_layers):
        row = cache.kv_heads_for(layer) * cache.head_dim_for(layer)
        for base in range(0, n_tokens, chunk):
            n = min(chunk, n_tokens - base)
            ks = torch.randn((n, row), device="cuda", generator=g)
            vs = torch.randn((n, row), device="cuda", generator=g)
            if outliers:
                for x in (ks, vs):
                    x.mul_(0.5)
                    hit = torch.rand(x.shape, device="cuda", generator=g) < 0.01
                    sign = torch.where(torch.rand(x.shape, device="cuda", generator=g) < 0.5, -40.0, 40.0)
                    x.copy_(torch.where(hit, sign, x))
            else:
                ks, vs = ks.half().float(), vs.half().float()
            fwd.b_step_kv_write(layer, base, n, ks, vs)
    torch.cuda.synchronize()


# The V buffer starts 256 bytes into its allocation, as in the caches vfkv_cache_create allocates itself: K and V
# of one row then differ in address bits 7-8 (see the comment there).
V_SKEW = 256


STEP_SPREAD = {}   # filled by time_steps: percentiles of single event-timed steps, microseconds


def time_steps(torch, step, args, rotating=False):
    """W untimed steps, then exactly K timed steps between two device synchronisations.  One step's
    launches are captured once into a HIP graph and replayed, so the host's per-launch cost (Python
    and ctypes here) does not gate a step that is only a few hundred microseconds of GPU work.
    rotating: steps of a handful of launches (fewer than 8 layers).  Replaying a graph of one or two kernels measures
    the graph launch, not the kernels, so all K steps are captured into ONE graph -- step(i) works on cache instance
    i % 4, so that no step finds its rows in a cache -- and the timed region is one replay of it (the warm-up is another
    replay: K >= W steps)."""
    if rotating and not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step(0)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(args.steps):
                step(i)
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        mean = (time.perf_counter() - t0) / args.steps
        stream = torch.cuda.current_stream()
        pairs = []
        for _ in range(20):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            graph.replay()
            e1.record(stream)
            pairs.append((e0, e1))
        torch.cuda.synchronize()
        us = sorted(e0.elapsed_time(e1) * 1e3 / args.steps for e0, e1 in pairs)
        STEP_SPREAD.clear()
        STEP_SPREAD.update({"p10": us[2], "p50": us[10], "p90": us[18], "samples": 20,
                            "note": f"per step of {args.steps}-step graph replays"})
        return mean
    if rotating:
        step0 = step
        counter = [0]
        def step():
            step0(counter[0])
            counter[0] += 1
    run = step
    if not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()                       # first-use initialisation must not happen under capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        run = graph.replay
    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    mean = (time.perf_counter() - t0) / args.steps
    # spread of single steps: every replay bracketed by its own pair of events, after the timed region above
    n = min(max(args.steps, 20), 200)
    pairs = []
    stream = torch.cuda.current_stream()
    for _ in range(n):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        run()
        e1.record(stream)
        pairs.append((e0, e1))
    torch.cuda.synchronize()
    us = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in pairs)
    STEP_SPREAD.clear()
    STEP_SPREAD.update({"p10": us[n // 10], "p50": us[n // 2], "p90": us[(n * 9) // 10], "samples": n})
    return mean


def bench_decode(args, wl):
    import torch

    import vulkanforge_amd as vf
    from vulkanforge_amd import _ffi

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, H, Hkv, D = wl.n_layers, wl.n_heads, wl.n_kv_heads, wl.head_dim
    max_seq = wl.context
    es = wl.dtype.element_size()
    # A model of fewer than 8 layers is a step of a handful of launches: it is timed as K steps inside one graph, each on
    # one of four cache instances in rotation (instance r = layers [r L, (r + 1) L) of one larger cache)
    rotating = L < 8
    inst = 4 if rotating else 1
    nbytes = L * inst * max_seq * Hkv * D * es
    kbuf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    vbuf = torch.empty(nbytes + V_SKEW, dtype=torch.uint8, device=dev)[V_SKEW:]
    cache = vf.KvCache(vf.KvCacheConfig(L * inst, Hkv, D, max_seq, dtype=wl.dtype), k_buffer=kbuf.data_ptr(),
                       v_buffer=vbuf.data_ptr())
    fwd = vf.Forward(cache, H)
    outliers = wl.name == "decode_fp8_8k_32layers"

    class _AllInstances:
        n_layers = L * inst
    fill_cache(torch, vf, fwd, _AllInstances, max_seq, args.seed, outliers)

    g = torch.Generator(device="cuda").manual_seed(args.seed + 1)
    q = torch.randn((L, H, D), device=dev, generator=g)
    if not args.f32_queries:
        q = q.half().float()
    o = torch.zeros((L, H, D), device=dev)
    k_new = torch.randn((L, Hkv * D), device=dev, generator=g).half().float()
    v_new = torch.randn((L, Hkv * D), device=dev, generator=g).half().float()
    pos = wl.context - 1
    scale = 1.0 / (D ** 0.5)
    starts = [_ffi.lib().vfkv_kv_start_decode(pos, wl.layer_window(i)) if wl.layer_window(i) else 0 for i in range(L)]

    gate = torch.randn((L, H * D), device=dev, generator=g) if wl.gated else None

    def step_gate_separate():   # step_attention, then step_attn_gated_output as a launch of its own
        for layer in range(L):
            fwd.run_scalar_attn(layer, pos, q[layer], o[layer], kv_start=starts[layer], scale=scale, softcap=wl.softcap)
            fwd.run_sigmoid_mul(gate[layer], o[layer], H * D, H * D, H * D, 0)

    rope_kw = None
    if wl.rope:
        import oracle as _o
        rope_kw = dict(q_norm_weight=(1 + 0.1 * torch.randn(D, device=dev, generator=g)), k_norm_weight=(1 + 0.1 * torch.randn(D, device=dev, generator=g)),
                       eps=1e-6)
        theta_scale = float(_o.rope_theta_scale(10000.0, D))
        q_rot = torch.zeros((L, H, D), device=dev)

    def step_rope_separate():   # QNormRope + KNormRope + KvWrite as one launch, then attention (split + merge)
        for layer in range(L):
            fwd.step_qk_rope_kv_write(layer, pos, 1, q[layer], k_new[layer], v_new[layer], D, theta_scale, q_out=q_rot[layer], **rope_kw)
            fwd.run_scalar_attn(layer, pos, q_rot[layer], o[layer], kv_start=starts[layer], scale=scale, softcap=wl.softcap)

    def step(i=0):
        base = (i % inst) * L       # first layer of the cache instance this step works on
        for layer in range(L):
            if wl.rope:         # norm + RoPE of the token's Q and K rows, append and attention in one call
                fwd.step_qk_rope_kv_write_attention(base + layer, pos, q[layer], k_new[layer], v_new[layer], o[layer], D, theta_scale,
                                                    kv_start=starts[layer], scale=scale, softcap=wl.softcap, **rope_kw)
            elif wl.gated:        # step_attention + step_attn_gated_output: the merge applies the gate
                fwd.step_attention_gated(base + layer, pos, q[layer], o[layer], gate[layer], H * D, H * D, 0,
                                         k_src=k_new[layer] if wl.append else None, v_src=v_new[layer] if wl.append else None,
                                         kv_start=starts[layer], scale=scale, softcap=wl.softcap)
            elif wl.append:     # step_kv_write + step_attention of the new token, issued as one call
                fwd.step_kv_write_attention(base + layer, pos, q[layer], k_new[layer], v_new[layer], o[layer],
                                            kv_start=starts[layer], scale=scale, softcap=wl.softcap)
            else:
                fwd.run_scalar_attn(base + layer, pos, q[layer], o[layer], kv_start=starts[layer], scale=scale,
                                    softcap=wl.softcap)

    gate_separate_us = time_steps(torch, step_gate_separate, args) * 1e6 if wl.gated and not wl.append else None
    rope_separate_us = time_steps(torch, step_rope_separate, args) * 1e6 if wl.rope else None
    sec_per_step = time_steps(torch, step, args, rotating=rotating)
    step_spread = dict(STEP_SPREAD)
    bytes_step = wl.kv_bytes_step()

    # ---- duration of the split worker (the dominant kernel): its launches of one step, back to back on
    # the benchmark's stream, bracketed by one pair of HIP events; repeated and averaged.  (Events around
    # every single launch would add their own packets between kernels and overstate the duration.)
    stream = torch.cuda.current_stream()
    lib = _ffi.lib()
    max_tiles = (max_seq + 63) // 64
    so = torch.empty((H * max_tiles * D,), device=dev)
    sm = torch.empty((H * max_tiles,), device=dev)
    ss = torch.empty((H * max_tiles,), device=dev)

    # (fewer than 8 layers: the launches of at least 32 steps over the rotating cache instances, so that the pair of events
    # brackets kernels and not one graph launch)
    split_reps = (32 + L - 1) // L if rotating else 1

    def split_only():
        for rep in range(split_reps):
            for layer in range(L):
                span = wl.context - starts[layer]
                tile = lib.vfkv_decode_tile_for(span, H, Hkv, D, int(wl.dtype))
                # the step's own launch starts at the tile that holds kv_start; the standalone split call numbers its tiles
                # from row 0 (flash_attn_split.comp), so a windowed layer is handed the slab from that tile on
                skip = starts[layer] // tile * tile
                phys = (rep % inst) * L + layer
                klay = cache.k_ptr + cache.layer_offset_bytes(phys) + skip * cache.row_bytes(phys)
                vlay = cache.v_ptr + cache.layer_offset_bytes(phys) + skip * cache.row_bytes(phys)
                fwd.run_flash_attn_split(q[layer], klay, vlay, wl.dtype, so, sm, ss, H, Hkv, D, wl.context - skip, scale,
                                         kv_start=starts[layer] - skip, tile=tile, softcap=wl.softcap, interleaved=True)

    def event_timed(fn, reps):
        """Total milliseconds of `reps` replays of fn's launches (captured once into a graph) between two events."""
        run = fn
        if not args.no_graph:
            fn()
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                fn()
            run = gr.replay
        run()
        torch.cuda.synchronize()
        evs = []
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            run()
            e1.record(stream)
            evs.append((e0, e1))
        torch.cuda.synchronize()
        return sum(e0.elapsed_time(e1) for e0, e1 in evs)

    n_ev = min(max(args.steps, 5), 20)
    split_ms = event_timed(split_only, n_ev)
    launches = n_ev * L * split_reps
    bytes_launch = bytes_step / L          # mean over the layers of the step
    avg_ms = split_ms / launches
    achieved = bytes_launch / (avg_ms * 1e-3) / 1e9

    # ---- what the same bytes cost without any arithmetic, timed the same way over the same slabs (compute-free kernels
    # of libvfkv_calib.so): a plain contiguous read, the worker's own walk and request pattern, and an empty launch of
    # the worker's grid.  Only for the geometry the pattern kernel is written for (FP8 rows, head_dim 128, no window).
    floors = None
    if wl.dtype.label() == "FP8" and D == 128 and not wl.window:
        import ctypes as C
        calib_path = os.path.join(ROOT, "vulkanforge_amd", "libvfkv_calib.so")
        if not os.path.exists(calib_path):
            raise ImportError(f"{calib_path} is missing: build it with `make -C vulkanforge_amd/csrc`")
        calib = C.CDLL(calib_path)
        calib.vfkv_calib_stream_read.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]
        calib.vfkv_calib_pattern_read.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        calib.vfkv_calib_empty.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        sink = torch.zeros(1024, dtype=torch.int32, device=dev)
        tile = lib.vfkv_decode_tile_for(wl.context, H, Hkv, D, int(wl.dtype))
        n_tiles = (wl.context + tile - 1) // tile
        layer_bytes = wl.context * Hkv * D * es

        def per_layer(call):
            def run():
                st = torch.cuda.current_stream().cuda_stream
                for layer in range(L):
                    kp = cache.k_ptr + cache.layer_offset_bytes(layer)
                    vp = cache.v_ptr + cache.layer_offset_bytes(layer)
                    rc = call(kp, vp, st)
                    assert rc == 0, rc
            return run

        stream_us = event_timed(per_layer(lambda kp, vp, st: calib.vfkv_calib_stream_read(kp, vp, layer_bytes // 16 * 16, sink.data_ptr(), st)), n_ev) * 1e3 / (n_ev * L)
        pattern_us = event_timed(per_layer(lambda kp, vp, st: calib.vfkv_calib_pattern_read(kp, vp, wl.context, Hkv, n_tiles, sink.data_ptr(), st)), n_ev) * 1e3 / (n_ev * L)
        empty_us = event_timed(per_layer(lambda kp, vp, st: calib.vfkv_calib_empty(Hkv, n_tiles, sink.data_ptr(), st)), n_ev) * 1e3 / (n_ev * L)
        floors = {"stream_floor_us": stream_us, "pattern_floor_us": pattern_us, "empty_launch_us": empty_us}

    mfma_worker = mfma_decode_worker(wl.dtype.label(), D)
    f32_mfma = wl.dtype.label() == "FP32" and (D in (64, 128, 256) or (64 < D < 256 and D % 16 == 0)) and os.environ.get("VFKV_DECODE_WORKER", "m")[:1] != "v"
    il_worker = mfma_worker and D in (64, 128, 256) and os.environ.get("VFKV_DECODE_IL", "1")[:1] != "0"   # (mirrors split_interleaves() of the library)
    worker_name = (("split_mfma_il_rope_kernel" if wl.rope else "split_mfma_il_kernel") if il_worker else "split_mfma_kernel" if mfma_worker
                   else "split_mfma_f32_kernel" if f32_mfma else "split_kernel")
    traffic, traffic_source = profiled_traffic(wl.name) if mfma_worker else (None, None)   # the profiles cover the default worker
    result = {
        "metric": "kv_read_GBps_decode_step",
        "value": bytes_step / sec_per_step / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec_per_step * 1e3,
        "us_per_decode_step": sec_per_step * 1e6,
        "step_us_event_timed": step_spread,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": MFMA_DTYPE if mfma_worker else "f32 mfma, f32 accumulate" if f32_mfma else "f32",
        "kv_dtype": wl.dtype.label(),
        "launch": "eager" if args.no_graph else "hip_graph",
        "data": "synthetic, seeded N(0,1); queries " + ("general f32" if args.f32_queries else "cast to fp16 as the configuration states") + "; K/V rows cast to fp16 and written through the append kernels",
        "config": {"workload": wl.name, "n_layers": L, "n_heads": H, "n_kv_heads": Hkv, "head_dim": D,
                   "context": wl.context, "append_per_step": wl.append, "kv_bytes_per_step": bytes_step,
                   "pct_of_hbm_peak": 100.0 * bytes_step / sec_per_step / 1e9 / HBM_PEAK_GBPS},
        "roofline": {"bound": "hbm", "kernel": worker_name, "achieved": achieved, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic, "traffic_source": traffic_source,
                     "avg_launch_us": avg_ms * 1e3, "launches_timed": launches,
                     "algorithmic_bytes_per_launch": bytes_launch},
    }
    if floors is not None:   # same bytes, same slabs, same timing method, no arithmetic
        result["roofline"].update(floors)
        result["roofline"]["frac_of_pattern_floor"] = floors["pattern_floor_us"] / (avg_ms * 1e3)

    if gate_separate_us is not None:
        result["config"]["us_per_step_with_separate_gate_launch"] = gate_separate_us
    if rope_separate_us is not None:
        result["config"]["us_per_step_with_separate_rope_append_launch"] = rope_separate_us

    if not args.no_cpu_baseline:
        import numpy as np

        import oracle
        threads = len(os.sched_getaffinity(0))
        per_layer = L * max_seq * Hkv * D * es // L
        done_bytes, spent, layers_done = 0, 0.0, 0
        if rotating:        # the timed steps ended on some cache instance: one more step on instance 0, which the oracle reads below
            step(0)
            torch.cuda.synchronize()
        for layer in range(L):
            lo = layer * per_layer
            kh = kbuf[lo:lo + per_layer].cpu().numpy().view(oracle.NP_DTYPE[int(wl.dtype)]).reshape(max_seq, Hkv, D)
            vh = vbuf[lo:lo + per_layer].cpu().numpy().view(oracle.NP_DTYPE[int(wl.dtype)]).reshape(max_seq, Hkv, D)
            qh = (q_rot if wl.rope else q)[layer].cpu().numpy()      # (rope: the rotated queries that the separate launch left)
            c0 = time.perf_counter()
            ref = oracle.attn_decode_ref(qh, kh, vh, int(wl.dtype), H, Hkv, D, wl.context, scale,
                                         kv_start=starts[layer], softcap=wl.softcap, threads=threads)
            if wl.gated:
                ref = oracle.sigmoid_mul(gate[layer].cpu().numpy(), ref.reshape(-1), H * D, H * D, 0).reshape(H, D)
            spent += time.perf_counter() - c0
            done_bytes += wl.kv_bytes_layer(layer)
            layers_done += 1
            if layer == 0:   # the timed GPU output of this layer also has to agree with the oracle
                err = float(np.abs(o[layer].cpu().numpy() - ref).max())
                result["config"]["max_abs_err_vs_oracle_layer0"] = err
            if spent >= args.cpu_seconds:
                break
        result["cpu_baseline"] = {"value": done_bytes / spent / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                                  "sample": f"{layers_done} of {L} layers of the same step, CPU oracle "
                                            f"(attn_decode_ref, f64 accumulation), {spent:.1f} s", **host_cpu()}
    cache.destroy()
    return result


def bench_prefill(args, wl):
    import torch

    import vulkanforge_amd as vf

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, H, Hkv, D = wl.n_layers, wl.n_heads, wl.n_kv_heads, wl.head_dim
    max_seq = wl.base_pos + wl.m
    es = wl.dtype.element_size()
    per_layer = max_seq * Hkv * D * es
    kbuf = torch.empty(L * per_layer, dtype=torch.uint8, device=dev)
    vbuf = torch.empty(L * per_layer + V_SKEW, dtype=torch.uint8, device=dev)[V_SKEW:]
    cache = vf.KvCache(vf.KvCacheConfig(L, Hkv, D, max_seq, dtype=wl.dtype), k_buffer=kbuf.data_ptr(),
                       v_buffer=vbuf.data_ptr())
    fwd = vf.Forward(cache, H)
    if wl.workspace:                  # sized for a serving context, as the decode path has it
        fwd.workspace = vf.Workspace(H, D, max(max_seq, 32768))

    class _W:  # fill_cache only needs n_layers
        n_layers = L
    fill_cache(torch, vf, fwd, _W, wl.base_pos, args.seed, False)
    g = torch.Generator(device="cuda").manual_seed(args.seed + 1)
    q = torch.randn((wl.m, H, D), device=dev, generator=g)
    if not args.f32_queries:
        q = q.half().float()
    kn = torch.randn((wl.m, Hkv * D), device=dev, generator=g).half().float()
    vn = torch.randn((wl.m, Hkv * D), device=dev, generator=g).half().float()
    o = torch.zeros((wl.m, H, D), device=dev)
    qgate = torch.randn((wl.m, H, 2, D), device=dev, generator=g) if wl.gated else None   # per (token, head): [Q | G]

    def attention(layer):
        if wl.gated:   # b_step_attention + b_step_attn_gated_output: the attention kernel's store applies the gate
            fwd.b_step_attention_gated(layer, wl.base_pos, wl.m, q, o, qgate, D, 2 * D, D)
        else:
            fwd.b_step_attention(layer, wl.base_pos, wl.m, q, o, use_workspace=wl.workspace)

    def step():
        for layer in range(L):
            fwd.b_step_kv_write(layer, wl.base_pos, wl.m, kn, vn)
            attention(layer)

    def step_gate_separate():   # the gate as a launch of its own after the attention
        for layer in range(L):
            fwd.b_step_kv_write(layer, wl.base_pos, wl.m, kn, vn)
            fwd.b_step_attention(layer, wl.base_pos, wl.m, q, o)
            fwd.b_step_attn_gated_output(o, qgate, wl.m, D)

    def step_with(**opts):      # the same step with options of the call (VFKV_PREFILL_F16_WEIGHTS / VFKV_PREFILL_FP8_SCORES)
        def run():
            for layer in range(L):
                fwd.b_step_kv_write(layer, wl.base_pos, wl.m, kn, vn)
                fwd.b_step_attention(layer, wl.base_pos, wl.m, q, o, use_workspace=wl.workspace, **opts)
        return run

    gate_separate_ms = time_steps(torch, step_gate_separate, args) * 1e3 if wl.gated else None
    f16w = None
    if not wl.gated and D == 128 and wl.dtype.label() in ("FP8", "FP16"):
        f16w = {}
        variants = [("f16_weights", dict(f16_weights=True))]
        if wl.dtype.label() == "FP8":
            variants += [("fp8_scores", dict(fp8_scores=True)), ("f16_weights+fp8_scores", dict(f16_weights=True, fp8_scores=True))]
        if args.f32_queries:     # general f32 queries: what rounding them to f16 inside the call saves (the remainder pass)
            variants += [("f16_queries", dict(f16_queries=True))]
        for name, opts in variants:
            ms = time_steps(torch, step_with(**opts), args) * 1e3
            f16w[name] = {"ms_per_step": ms, "TFLOPs": wl.flops_layer() * L / (ms * 1e-3) / 1e12}
            if not args.no_cpu_baseline:        # the error of the option's output against the oracle is taken below
                f16w[name]["_o_last_rows"] = o[wl.m - 8:].clone()
    sec_per_step = time_steps(torch, step, args)
    step_spread = dict(STEP_SPREAD)
    flops_step = wl.flops_layer() * L

    # ---- duration of the attention kernel (the dominant kernel): the step's attention launches without the appends, back
    # to back on the benchmark's stream (one graph), bracketed by one pair of HIP events per replay and averaged, as the
    # decode workloads time their worker.  (Events around every single launch add their own packets between the kernels.)
    stream = torch.cuda.current_stream()

    def attention_only():
        for layer in range(L):
            attention(layer)

    run = attention_only
    if not args.no_graph:
        attention_only()
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            attention_only()
        run = gr.replay
    run()
    torch.cuda.synchronize()
    pairs = []
    n_ev = min(max(args.steps, 5), 20)
    for _ in range(n_ev):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        run()
        e1.record(stream)
        pairs.append((e0, e1))
    torch.cuda.synchronize()
    launches = n_ev * L
    avg_ms = sum(a.elapsed_time(b) for a, b in pairs) / launches
    achieved = wl.flops_layer() / (avg_ms * 1e-3) / 1e12
    f32_cache = wl.dtype.label() == "FP32"
    peak = MFMA_F32_PEAK_TFLOPS if f32_cache else MFMA_F16_PEAK_TFLOPS
    traffic, traffic_source = profiled_traffic(wl.name)
    result = {
        "metric": "prefill_attention_TFLOPs",
        "value": flops_step / sec_per_step / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec_per_step * 1e3,
        "step_us_event_timed": step_spread,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32 mfma" if f32_cache else MFMA_DTYPE,
        "kv_dtype": wl.dtype.label(),
        "data": "synthetic, seeded N(0,1); queries " + ("general f32" if args.f32_queries else "cast to fp16 as the configuration states") + "; K/V rows cast to fp16 and written through the append kernels",
        "config": {"workload": wl.name, "n_layers": L, "n_heads": H, "n_kv_heads": Hkv, "head_dim": D,
                   "m": wl.m, "q_start": wl.base_pos, "n_kv": max_seq, "flop_per_step": flops_step},
        "roofline": {"bound": "mfma", "kernel": prefill_kernel_name(wl.dtype.label(), D, H // Hkv),
                     "achieved": achieved, "peak": peak,
                     "unit": "TFLOP/s", "frac": achieved / peak, "traffic": traffic, "traffic_source": traffic_source,
                     "avg_launch_us": avg_ms * 1e3, "launches_timed": launches,
                     "algorithmic_flop_per_launch": wl.flops_layer()},
    }
    if gate_separate_ms is not None:
        result["config"]["ms_per_step_gate_as_separate_launch"] = gate_separate_ms
    if f16w is not None:          # options of the call, not what `value` is measured with
        result["config"]["with_options"] = f16w
    if not args.no_cpu_baseline:
        import numpy as np

        import oracle
        threads = len(os.sched_getaffinity(0))
        last = (L - 1) * per_layer   # `o` holds the output of the last layer of the step
        kh = kbuf[last:last + per_layer].cpu().numpy().view(oracle.NP_DTYPE[int(wl.dtype)]).reshape(max_seq, Hkv, D)
        vh = vbuf[last:last + per_layer].cpu().numpy().view(oracle.NP_DTYPE[int(wl.dtype)]).reshape(max_seq, Hkv, D)
        ms = 8                       # the last `ms` query rows of that layer, repeated until the time target
        qs = wl.base_pos + wl.m - ms
        qh = q[wl.m - ms:].cpu().numpy()
        flops_sample = sum(qs + i + 1 for i in range(ms)) * H * 4 * D
        spent, reps, ref = 0.0, 0, None
        while spent < args.cpu_seconds and reps < 1024:
            c0 = time.perf_counter()
            ref = oracle.attn_batch_ref(qh, kh, vh, int(wl.dtype), ms, max_seq, H, Hkv, D, qs, 1.0 / D ** 0.5,
                                        threads=threads)
            if wl.gated:
                ref = oracle.sigmoid_mul(qgate[wl.m - ms:].cpu().numpy().reshape(-1), ref.reshape(-1), D, 2 * D, D).reshape(ms, H, D)
            spent += time.perf_counter() - c0
            reps += 1
        err = float(np.abs(o[wl.m - ms:].cpu().numpy() - ref).max())
        result["config"]["max_abs_err_vs_oracle_last_rows"] = err
        for v in (f16w or {}).values():
            v["max_abs_err_vs_oracle_last_rows"] = float(np.abs(v.pop("_o_last_rows").cpu().numpy() - ref).max())
        result["cpu_baseline"] = {"value": flops_sample * reps / spent / 1e12, "unit": "TFLOP/s", "cores": threads,
                                  "kind": "port",
                                  "sample": f"last {ms} of {wl.m} query rows of one layer, {reps} repetitions, CPU "
                                            f"oracle (attn_batch_ref, f64), {spent:.1f} s", **host_cpu()}
    cache.destroy()
    return result


def bench_rope_append(args, wl):
    """One step = for every layer one launch of K-norm + RoPE + append (K and V rows).  Also times the plain append
    of the same rows (no norm, no rotation) so the cost of the fused arithmetic can be read off."""
    import numpy as np
    import torch

    import vulkanforge_amd as vf

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, Hkv, D, T = wl.n_layers, wl.n_kv_heads, wl.head_dim, wl.n_tokens
    cache = vf.KvCache(vf.KvCacheConfig(L, Hkv, D, wl.base_pos + T, dtype=wl.dtype))
    fwd = vf.Forward(cache, Hkv)
    g = torch.Generator(device="cuda").manual_seed(args.seed)
    k = torch.randn((L, T, Hkv * D), device=dev, generator=g)
    v = torch.randn((L, T, Hkv * D), device=dev, generator=g).half().float()
    w = 1.0 + 0.1 * torch.randn((D,), device=dev, generator=g)
    theta_scale = float((1.0 / 1e6) ** (2.0 / D))

    def step():
        for layer in range(L):
            fwd.step_k_rope_kv_write(layer, wl.base_pos, T, k[layer], v[layer], D, theta_scale, k_norm_weight=w)

    def plain():
        for layer in range(L):
            fwd.b_step_kv_write(layer, wl.base_pos, T, k[layer], v[layer])

    H = 4 * Hkv                                      # query heads of the same token rows (GQA group of 4)
    qq = torch.randn((L, T, H * D), device=dev, generator=g)
    fwd_q = vf.Forward(cache, H)

    def qk():                                        # the Q rows in the same launch (QNormRope + KNormRope + KvWrite)
        for layer in range(L):
            fwd_q.step_qk_rope_kv_write(layer, wl.base_pos, T, qq[layer], k[layer], v[layer], D, theta_scale,
                                        q_norm_weight=w, k_norm_weight=w)

    sec = time_steps(torch, step, args)
    sec_plain = time_steps(torch, plain, args)
    sec_qk = time_steps(torch, qk, args)
    step()
    torch.cuda.synchronize()
    result = {
        "metric": "k_rope_append_GBps", "value": wl.bytes_step() / sec / 1e9, "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3, "us_per_launch": sec * 1e6 / L,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "kv_dtype": wl.dtype.label(),
        "data": "synthetic, seeded N(0,1)",
        "config": {"workload": wl.name, "n_layers": L, "n_kv_heads": Hkv, "head_dim": D, "tokens_per_layer": T,
                   "base_pos": wl.base_pos, "bytes_per_step": wl.bytes_step(),
                   "plain_append_us_per_launch": sec_plain * 1e6 / L,
                   "with_32_query_heads_us_per_launch": sec_qk * 1e6 / L},
        "roofline": {"bound": "hbm", "kernel": "rope_append_kernel", "achieved": wl.bytes_step() / sec / 1e9,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": wl.bytes_step() / sec / 1e9 / HBM_PEAK_GBPS,
                     "traffic": None, "avg_launch_us": sec * 1e6 / L},
    }
    if not args.no_cpu_baseline:
        import oracle
        kk = k[0].cpu().numpy().reshape(T, Hkv, D)
        pos = (wl.base_pos + np.arange(T)).astype(np.int32)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < min(args.cpu_seconds, 2.0):
            ref = oracle.rms_norm_rope(kk, pos, D, D, theta_scale, weight=w.cpu().numpy(), eps=1e-6)
            enc = oracle.f32_to_e4m3(ref.reshape(-1)) if wl.dtype == vf.KvDtype.F8 else ref
            reps += 1
        spent = time.perf_counter() - t0
        result["cpu_baseline"] = {"value": wl.bytes_step() / L / 2 * reps / spent / 1e9, "unit": "GB/s",
                                  "cores": oracle.default_threads(), "kind": "port",
                                  "sample": f"K rows of one layer, {reps} repetitions, CPU oracle, {spent:.1f} s"}
        del enc
    cache.destroy()
    return result


def copy_calibration(args):
    """Plain device-to-device copy of a known size, launched `steps` times: the reference point for the
    FETCH_SIZE / WRITE_SIZE counters (what they read for a kernel whose HBM traffic is known)."""
    import torch
    n = 64 << 20
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
    bufs = [torch.empty_like(src) for _ in range(8)]      # rotate destinations so nothing stays cached
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        bufs[i % len(bufs)].copy_(src)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return {"metric": "copy_calibration", "bytes_read_per_launch": n, "bytes_written_per_launch": n,
            "launches": args.steps, "value": 2 * n * args.steps / dt / 1e9, "unit": "GB/s", "n_gpus": 1}


HEADLINE = "decode_fp8_32k_32layers"
# the other benchmark configurations, run briefly after the headline workload so that one invocation witnesses all five
OTHER_CONFIGS = ("decode_f16_2k_1layer", "decode_fp8_8k_32layers", "decode_f16_hd256_sliding_12layers",
                 "prefill_fp8_512x4608_32layers")


def run_workload(args, name):
    from vulkanforge_amd import workloads
    if name in workloads.DECODE:
        return bench_decode(args, workloads.DECODE[name])
    if name in workloads.PREFILL:
        return bench_prefill(args, workloads.PREFILL[name])
    if name in workloads.ROPE_APPEND:
        return bench_rope_append(args, workloads.ROPE_APPEND[name])
    if name == "copy_calibration":
        return copy_calibration(args)
    return None


def summary(res):
    """The fields of a workload's own JSON line that the headline line carries along in its 'workloads' array."""
    cfg, roof = res["config"], res["roofline"]
    err = cfg.get("max_abs_err_vs_oracle_layer0", cfg.get("max_abs_err_vs_oracle_last_rows"))
    out = {"workload": cfg["workload"], "ms_per_step": res["ms_per_step"], "steps": res["steps"], "value": res["value"],
           "unit": res["unit"], "kv_dtype": res["kv_dtype"],
           "roofline": {k: roof[k] for k in ("kernel", "bound", "frac", "avg_launch_us", "achieved", "peak", "unit") if k in roof},
           "max_abs_err_vs_oracle": err}
    for k in ("stream_floor_us", "pattern_floor_us", "empty_launch_us"):
        if k in roof:
            out["roofline"][k] = roof[k]
    if "cpu_baseline" in res:
        out["cpu_baseline"] = {k: res["cpu_baseline"][k] for k in ("value", "unit", "cores")}
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}): this build has no multi-GPU path.",
              file=sys.stderr)
        sys.exit(2)
    from vulkanforge_amd import workloads
    res = run_workload(args, args.workload)
    if res is None:
        print("unknown workload; choose from: " + ", ".join(list(workloads.DECODE) + list(workloads.PREFILL) + list(workloads.ROPE_APPEND) + ["copy_calibration"]),
              file=sys.stderr)
        sys.exit(2)
    if args.workload == HEADLINE and not args.no_other_workloads:
        import copy
        brief = copy.copy(args)
        brief.cpu_seconds = min(args.cpu_seconds, 1.0)
        res["workloads"] = []
        for name in OTHER_CONFIGS:
            brief.steps = min(args.steps, 5 if name in workloads.PREFILL else 30)
            brief.warmup = min(args.warmup, 2 if name in workloads.PREFILL else 10)
            res["workloads"].append(summary(run_workload(brief, name)))
    print(json.dumps(res))


if __name__ == "__main__":
    main()

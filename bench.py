#!/usr/bin/env python3
"""Headline benchmark: fused decode-GEMV at batch 1 on Qwen-27B-like MLP shapes.

One step = one pass of the hot path over the three coded MLP matrices of a layer
(gate and up: 17408x5120, down: 5120x17408) on seeded synthetic BF16 weights
(N(0,0.02) with per-row log-normal(0,0.5) scale and 0.1% outliers at 10x) against
an N(0,1) BF16 activation vector: gate and up take the same vector and run as one
fused decode-GEMV launch, down as another (--no-groups: three launches).  The three
matrices together are ~354 MB coded, more than L2 + Infinity Cache, so every step
streams its compressed bytes from HBM.

Prints ONE JSON line: metric = compressed bytes consumed per second (GB/s), with
the achieved fraction of the 8 TB/s HBM roofline for the dominant kernel and a
CPU baseline (the CPU oracle's decode + matvec on the host cores).

After the warm-up, K eager steps give the per-launch durations (HIP events on the
launch stream); the K timed steps are then replays of one HIP graph of a step
(--no-graph times the eager steps instead).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0
LAST_LEVEL_CACHE_BYTES = 256 << 20  # MI355X: 256 MB behind the L2s
MODEL_BF16_BYTES = 55_586_113_293  # dense BF16 bytes of the 27B model one token has to read at batch 1
SHAPES = {"gate": (17408, 5120), "up": (17408, 5120), "down": (5120, 17408)}
# one layer of the whole-stack workload: attention projections, then the MLP
LAYER = {"q": (6144, 5120), "k": (1024, 5120), "v": (1024, 5120), "o": (5120, 6144),
         "gate": (17408, 5120), "up": (17408, 5120), "down": (5120, 17408)}


def log(*a):
    print("[bench]", *a, file=sys.stderr, flush=True)


def bf16_words(values):
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def synth_weights(index, rows, cols):
    rng = np.random.default_rng(1000 + index)
    out = np.empty((rows, cols), dtype=np.uint16)
    scale = rng.lognormal(0.0, 0.5, size=(rows, 1)).astype(np.float32)
    step = 2048
    for lo in range(0, rows, step):  # chunked so the float temporaries stay small
        hi = min(rows, lo + step)
        w = rng.normal(0.0, 0.02, size=(hi - lo, cols)).astype(np.float32) * scale[lo:hi]
        mask = rng.random((hi - lo, cols)) < 1e-3
        w = np.where(mask, w * np.float32(10.0), w)
        out[lo:hi] = bf16_words(w)
    return out


GEMV_UP_TO = 2  # rows linear() gives to the vector-ALU kernel; read from HipContextTensor once it is imported


def algorithmic_bytes(t, m):
    """Bytes one fused GEMV launch has to touch once: both streams, the fused index,
    the per-class lookup tables, labels, activations and outputs."""
    b = t.buffers
    n = lambda k: b[k].numel() * b[k].element_size()
    rows, cols = t.shape
    # (the resident residual array starts every row class on a multiple of 16 rows: the rows it
    # holds beyond the matrix's are never read and are not counted)
    payload = t._main_bytes + min(n("residual_stream"), rows * cols * 3 // 4)
    _, tile_rows, tile_class, _ = t._tiling(m) if m <= GEMV_UP_TO else t._gemm_tiling()
    index = (n("fused_seg_state") + n("fused_seg_offset") + tile_rows.numel() * tile_rows.element_size()
             + tile_class.numel() * tile_class.element_size() + (n("row_pos") if "row_pos" in b else 0))
    tables = n("fused_lut") + n("fused_tab")
    labels = cols
    io = m * cols * 2 + m * rows * 2
    return dict(total=payload + index + tables + labels + io, payload=payload, index=index, tables=tables)


def host_description():
    model = ""
    try:
        for line in Path("/proc/cpuinfo").read_text().splitlines():
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"cpu": model, "logical_cpus": os.cpu_count(), "oracle_flags": "gcc -O3 (oracle/Makefile)"}


def measured_copy_gbps(torch):
    """Device-to-device copy of 1 GiB (read + write counted), the achievable HBM rate on this
    box next to the 8 TB/s nameplate."""
    src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    dst.copy_(src)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(5):
        dst.copy_(src)
    b.record()
    torch.cuda.synchronize()
    return 5 * 2 * src.numel() / (a.elapsed_time(b) * 1e-3) / 1e9


def reference_core():
    """The reference's own C++ coder, compiled from its sources into oracle/_ref by the oracle's
    Makefile; None where that build is absent."""
    import ctypes
    path = ROOT / "oracle" / "_ref" / "libref_context.so"
    if not path.exists():
        return None
    L = ctypes.CDLL(str(path))
    U8P, U16P, U32P = (ctypes.POINTER(t) for t in (ctypes.c_uint8, ctypes.c_uint16, ctypes.c_uint32))
    sz, u32, u64 = ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint64
    L.bcx_decode.argtypes = [U8P, sz, u64, u32, u32, U8P, U8P, u32, u32, u32, U16P, U32P, U16P]
    L.bcx_unpack6.argtypes = [U8P, sz, u64, U16P]
    L.bcx_decode_compact.argtypes = L.bcx_decode.argtypes
    L.bcx_decode.restype = L.bcx_decode_compact.restype = L.bcx_unpack6.restype = ctypes.c_int
    return L


def reference_decode(L, orc, frame, compact=False):
    """A frame decoded by the reference's bcx_decode (full 65536-slot lookup per context) or
    bcx_decode_compact (binary search in the cumulative table), and bcx_unpack6; the container
    around them (header, inflate, digests) is read by the oracle's parser."""
    import ctypes
    import hashlib
    s = orc.bctx_sections(frame)
    if s["mode"] == 1:
        return s["raw"]
    rows, cols = s["shape"]
    n = rows * cols
    p = lambda a, t: a.ctypes.data_as(ctypes.POINTER(t))
    u8, u16, u32 = ctypes.c_uint8, ctypes.c_uint16, ctypes.c_uint32

    def entropy(stream, freq, kind, main):
        data = np.frombuffer(stream, dtype=np.uint8)
        out = np.empty(n, dtype=np.uint16)
        freq = np.ascontiguousarray(freq, dtype=np.uint32).ravel()
        fn = L.bcx_decode_compact if compact else L.bcx_decode
        rc = fn(p(data, u8), len(stream), n, rows, cols, p(s["rc"], u8), p(s["cc"], u8), s["nr"], s["nc"],
                kind, p(main, u16) if main is not None else None, p(freq, u32), p(out, u16))
        if rc:
            raise RuntimeError(f"reference bcx_decode failed ({rc})")
        return out

    main = entropy(s["main_stream"], s["main_freq"], 0, None)
    if s["mode"] == 128:
        residual = entropy(s["res_stream"], s["res_freq"], 1, main)
    else:
        raw = np.frombuffer(s["res_stream"], dtype=np.uint8)
        residual = np.empty(n, dtype=np.uint16)
        if L.bcx_unpack6(p(raw, u8), len(raw), n, p(residual, u16)):
            raise RuntimeError("reference bcx_unpack6 failed")
    out = np.ascontiguousarray(orc.join_words(main, residual).reshape(rows, cols))
    if hashlib.sha256(out.tobytes()).digest() != s["digest"]:
        raise RuntimeError("reference decode does not reproduce the frame's digest")
    return out


def cpu_baseline(frames, words_of, x_words, min_seconds=8.0, max_frames=12):
    """CPU decode + fp32 matvec of whole frames of the workload, one thread, as the reference
    decodes a frame; frames are taken in turn until min_seconds of work are done.  Timed with
    the reference's own compiled coder where oracle/_ref holds it (kind "reference"), and
    with the CPU oracle (kind "port"); the reference figure is the headline when present."""
    from oracle import codec_oracle as orc
    names = list(frames)

    def timed(decode, what, seconds=min_seconds):
        coded = produced = done = 0
        checksum = 0.0
        t0 = time.perf_counter()
        while done < max_frames and (done == 0 or time.perf_counter() - t0 < seconds):
            name = names[done % len(names)]
            dec = decode(frames[name])
            wf = (dec.astype(np.uint32) << 16).view(np.float32)
            xf = (x_words[dec.shape[1]][0].astype(np.uint32) << 16).view(np.float32)
            checksum += float(np.sum(wf @ xf))
            assert np.array_equal(dec, words_of[name]), "CPU decode is not bit-exact"
            coded += len(frames[name])
            produced += dec.nbytes
            done += 1
            del dec, wf
        dt = time.perf_counter() - t0
        return dict(value=round(coded / dt / 1e9, 4), unit="GB/s", cores=1,
                    sample=f"{done} whole frames in turn from {', '.join(names)} ({coded} coded bytes): frame parse + "
                           f"sha256 + {what} + bit-exact check + fp32 matvec in {dt:.1f}s "
                           f"({produced / dt / 1e6:.1f} MB/s of BF16 produced)",
                    checksum=checksum)

    port = dict(timed(orc.bctx_decode, "the oracle's full-LUT rANS decode of both streams", min_seconds / 2), kind="port")
    core = reference_core()
    if core is not None:
        result = dict(timed(lambda f: reference_decode(core, orc, f),
                            "the reference's bcx_decode (full LUT) of both streams, compiled from its sources"),
                      kind="reference")
        result["oracle_port"] = port
        result["compact_lookup"] = dict(timed(lambda f: reference_decode(core, orc, f, compact=True),
                                              "the reference's bcx_decode_compact (search in the cumulative table) of both "
                                              "streams, compiled from its sources", min_seconds / 2), kind="reference")
    else:
        result = port
    # the reference decodes one frame per thread: every host core with a frame of its own, once
    from concurrent.futures import ThreadPoolExecutor
    decode = (lambda f: reference_decode(core, orc, f)) if core is not None else orc.bctx_decode
    threads = max(1, min(os.cpu_count() or 1, 16))
    jobs = [names[i % len(names)] for i in range(threads)]
    t0 = time.perf_counter()
    with ThreadPoolExecutor(max_workers=threads) as pool:
        sizes = list(pool.map(lambda n: decode(frames[n]).nbytes, jobs))
    dt = time.perf_counter() - t0
    total = sum(len(frames[n]) for n in jobs)
    result["one_frame_per_thread"] = dict(value=round(total / dt / 1e9, 4), unit="GB/s", cores=threads,
                                          sample=f"{threads} frames decoded concurrently, one thread each, in "
                                                 f"{dt:.1f}s ({sum(sizes) / dt / 1e6:.1f} MB/s of BF16 produced)")
    return result


def run_predictive(args):
    """A 5120 x 17408 target coded (PPCX) against a reference that is the target plus N(0, 0.002)
    noise, as a loaded model serves it: the tensor keeps the 4-bit context plane of its
    reference from load on, so no reference is resident or decoded.  One step = the product of
    the coded target with `--batch` activation rows (default 96 = 16 users x (5 draft tokens
    + 1), the verify shape): the activations packed, then the fused GEMM (one row: the GEMV)."""
    import torch
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor

    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a ROCm GPU")
    m = args.batch or 96
    rows, cols = 5120, 17408
    target = synth_weights(2, rows, cols)
    noise = np.random.default_rng(5).normal(0, 0.002, size=target.shape).astype(np.float32)
    ref = bf16_words((target.astype(np.uint32) << 16).view(np.float32) + noise)
    del noise
    t0 = time.perf_counter()
    frame = ppcx.encode(target, ref)
    t = HipPredictiveTensor(frame, ref, stride=1024, device="cuda:0")
    if t.fused is None:
        sys.exit(f"bench.py: the frame is not eligible for the fused kernels: {t.fused_reason}")
    log(f"PPCX frame {len(frame)} B ({8 * len(frame) / target.size:.3f} bit/weight) mode {t.mode}; setup {time.perf_counter() - t0:.1f}s")
    copies = [(t, None)]
    for _ in range(2):  # three targets in rotation: more bytes than the caches hold
        copies.append((HipPredictiveTensor(frame, ref, stride=1024, device="cuda:0"), None))
    x = torch.from_numpy(bf16_words(np.random.default_rng(7).normal(0, 1, size=(m, cols)))).view(torch.bfloat16).cuda()

    def step():
        return [c.linear(r, x) for c, r in copies]

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    dense = torch.from_numpy(target).view(torch.bfloat16).cuda().float()
    want = torch.nn.functional.linear(x.float(), dense)
    scale = torch.nn.functional.linear(x.float().abs(), dense.abs())
    got = copies[0][0].linear(copies[0][1], x, check=True).float()
    if not bool((got - want).abs().le(1e-2 * want.abs().clamp_min(1e-3 * scale)).all()):
        sys.exit("bench.py: the fused product is outside 1e-2 of the dense product")
    del dense, want, scale, got
    events = []
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    for _ in range(args.steps):
        for c, r in copies:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            c.linear(r, x)
            b.record()
            events.append((a, b))
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    launch = "eager"
    if args.graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            graph.replay()
            torch.cuda.synchronize()
        except Exception as exc:
            log(f"graph capture failed ({exc}); reporting the eager steps")
        else:
            wall0 = time.perf_counter()
            for _ in range(args.steps):
                graph.replay()
            torch.cuda.synchronize()
            wall = time.perf_counter() - wall0
            launch = "hip graph replay"
    for c, _ in copies:
        if c.error.item():
            sys.exit("bench.py: decoder error word set")
    ms_product = float(np.mean([a.elapsed_time(b) for a, b in events]))
    # bytes one product has to touch once: everything the tensor keeps on the device (the coded
    # target, its index and tables, the 4-bit context plane of the reference), activations, outputs
    coded = t.resident_bytes
    alg = coded + m * cols * 2 + m * rows * 2
    ms_per_step = wall / args.steps * 1e3
    value = len(copies) * alg / (ms_per_step * 1e-3) / 1e9
    print(json.dumps({
        "metric": "compressed-weight decode-GEMV GB/s", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u32 rANS state / bf16 weights / fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": f"PPCX target 5120x17408 coded against a reference (target + N(0, 0.002)), product with "
                               f"{m} activation rows as served: contexts of the reference resident as a 4-bit plane, no "
                               f"dense reference; three targets in rotation", "batch": m, "launch": launch},
        "ms_per_product": round(ms_per_step / len(copies), 4), "ms_per_product_eager_events": round(ms_product, 4),
        "frame_bytes": len(frame), "resident_bytes": coded,
        "context_plane_bytes": target.size // 2,
        "algorithmic_bytes_per_product": alg, "tok_s_equiv_rows_per_s": round(m * len(copies) / (ms_per_step * 1e-3), 1),
        # per product: the step's wall time over its products (under a graph the launches follow one
        # another without host gaps; events around single eager launches, kept beside it, include them)
        "roofline": {"bound": "hbm", "achieved": round(value, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(value / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": ("grf::fused_wave_kernel<PpcxWalk, 1, SCAN>" if m == 1 else
                                "pack_activations_kernel + grf::fused_gemm_kernel / fused_gemm_wide_kernel<PpcxWalk, MT, SCAN>")
                               + " (a product's share of the step)"},
    }), flush=True)


def run_stack(args, as_dict=False):
    """Every coded linear of a 64-layer stack resident at once, one pass at batch 64.

    Each layer holds q, k, v, o, gate, up and down as BCTX frames.  `--distinct-layers`
    layers are generated and encoded from their own seeds; the others are device copies of
    those in rotation (their own buffers, so a pass streams every layer's bytes from HBM,
    but no further host encoding)."""
    import torch
    from concurrent.futures import ThreadPoolExecutor
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    global GEMV_UP_TO
    GEMV_UP_TO = HipContextTensor.GEMV_UP_TO

    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a ROCm GPU")
    m = args.batch or 64
    t0 = time.perf_counter()

    def coded(job):
        layer, j, name = job
        rows, cols = LAYER[name]
        return job, codec.encode(synth_weights(100 * layer + j, rows, cols))

    jobs = [(d, j, name) for d in range(args.distinct_layers) for j, name in enumerate(LAYER)]
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        frames = dict(pool.map(coded, jobs))
    log(f"encoded {len(jobs)} matrices in {time.perf_counter() - t0:.1f}s")
    t0 = time.perf_counter()
    base = {}
    for job in jobs:
        # one segment length for every matrix, so that q/k/v and gate/up can share a launch
        t = HipContextTensor(frames[job], stride=1024, device="cuda:0", fused_segment=64)
        if t.fused is None:
            sys.exit(f"bench.py: {job} is not eligible for the fused kernels: {t.fused_reason}")
        t._gemm_tiling()
        base[job] = t
    log(f"indexed and uploaded in {time.perf_counter() - t0:.1f}s")
    layers = []
    for i in range(args.layers):
        d = i % args.distinct_layers
        src = {name: base[(d, j, name)] for j, name in enumerate(LAYER)}
        layers.append(src if i < args.distinct_layers else {k: v.clone() for k, v in src.items()})
    for layer in layers:
        for t in layer.values():
            t._gemm_tiling() if m > GEMV_UP_TO else t._tiling(m)
    torch.cuda.synchronize()
    frame_bytes = sum(t.frame_bytes for layer in layers for t in layer.values())
    resident = sum(t.resident_bytes for layer in layers for t in layer.values())
    dense = sum(2 * r * c for r, c in LAYER.values()) * args.layers
    log(f"{args.layers} layers resident: {dense} BF16 bytes as {frame_bytes} frame bytes, {resident} device bytes; "
        f"torch reports {torch.cuda.memory_allocated()} allocated")

    rng = np.random.default_rng(7)
    x = {k: torch.from_numpy(bf16_words(rng.normal(0, 1, size=(m, k)))).view(torch.bfloat16).cuda()
         for k in {c for _, c in LAYER.values()}}

    # q, k, v read the same activations, gate and up too: each group is one launch
    from georefine_amd.bitexact_context_gpu import HipLinearGroup
    names = (("q", "k", "v"), ("o",), ("gate", "up"), ("down",))
    grouped = not args.no_groups
    groups = [[HipLinearGroup([layer[n] for n in g]) if grouped and len(g) > 1 else None for g in names]
              for layer in layers] if grouped else None
    torch.cuda.synchronize()

    def step():
        for i, layer in enumerate(layers):
            for j, g in enumerate(names):
                xin = x[LAYER[g[0]][1]]
                if grouped and len(g) > 1:
                    groups[i][j].linear(xin, batch_invariant=m > GEMV_UP_TO)
                else:
                    for name in g:
                        layer[name].linear(xin, batch_invariant=m > GEMV_UP_TO)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # per-launch durations of the first layer's kernels, on the stream they run on
    probes = {name: [] for name in LAYER}
    wall0 = time.perf_counter()
    for _ in range(args.steps):
        for i, layer in enumerate(layers):
            for name, t in layer.items():
                if i == 0:
                    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    a.record()
                t.linear(x[LAYER[name][1]], batch_invariant=m > GEMV_UP_TO)
                if i == 0:
                    b.record()
                    probes[name].append((a, b))
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    launch = "eager"
    if args.graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            graph.replay()
            torch.cuda.synchronize()
        except Exception as exc:
            log(f"graph capture failed ({exc}); reporting the eager steps")
        else:
            wall0 = time.perf_counter()
            for _ in range(args.steps):
                graph.replay()
            torch.cuda.synchronize()
            wall = time.perf_counter() - wall0
            launch = "hip graph replay"
    for layer in layers:
        for name, t in layer.items():
            if t.error.item():
                sys.exit(f"bench.py: decoder error word set for {name}")
    ms = {name: float(np.mean([a.elapsed_time(b) for a, b in ev])) for name, ev in probes.items()}
    alg = {name: algorithmic_bytes(layers[0][name], m) for name in LAYER}
    step_bytes = sum(algorithmic_bytes(t, m)["total"] for layer in layers[:args.distinct_layers] for t in layer.values())
    step_bytes = step_bytes * args.layers // args.distinct_layers
    ms_per_step = wall / args.steps * 1e3
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    dom = max(LAYER, key=lambda n_: ms[n_])
    achieved = alg[dom]["total"] / (ms[dom] * 1e-3) / 1e9
    kernel = kernel_name(False, m, False, 64)  # (of the ungrouped launch that took longest)
    result = {
        "metric": "compressed-weight decode-GEMV GB/s", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u32 rANS state / bf16 weights / fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": f"whole stack resident: {args.layers} layers x (q 5120->6144, k/v 5120->1024, o 6144->5120, "
                               f"gate/up 5120->17408, down 17408->5120), one pass through every coded linear at batch {m}; "
                               f"{dense / 1e9:.1f} GB of dense BF16 held as {frame_bytes / 1e9:.1f} GB of frames "
                               f"(no embedding or head matrix in the stack)",
                   "batch": m, "layers": args.layers, "distinct_layers": args.distinct_layers,
                   "linears": args.layers * len(LAYER), "launch": launch,
                   "launches": "q/k/v and gate/up grouped" if grouped else "one per linear"},
        "dense_bf16_bytes": dense, "frame_bytes": frame_bytes, "resident_device_bytes": resident,
        "algorithmic_bytes_per_step": step_bytes,
        "effective_bf16_GBps": round(dense / (ms_per_step * 1e-3) / 1e9, 2),
        "tok_s_equiv": round(m / (ms_per_step * 1e-3), 1),
        "pct_hbm_roofline": round(100 * value / HBM_PEAK_GBPS, 2),
        "per_kernel": {n_: {"ms": round(ms[n_], 4), "alg_bytes": alg[n_]["total"],
                            "GBps": round(alg[n_]["total"] / (ms[n_] * 1e-3) / 1e9, 2)} for n_ in LAYER},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None, "kernel": f"{kernel} on {dom}"},
    }
    if as_dict:  # as a key of the headline line: the fields that line carries itself are left out
        for key in ("metric", "unit", "n_gpus", "higher_is_better", "scaling", "vs_baseline", "dtype", "data"):
            result.pop(key)
        layers.clear()
        base.clear()
        groups = graph = None
        torch.cuda.empty_cache()
        return result
    print(json.dumps(result), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50, help="untimed steps first (the clocks of an idle GPU take "
                                                         "some milliseconds of work to come up)")
    ap.add_argument("--batch", type=int, default=None, help="activation rows (default 1 for mlp, the headline figure, and 64 for stack); 1..2 run the fused GEMV, more the fused GEMM")
    ap.add_argument("--segment", type=int, default=0, help="fused segment length (0 = automatic)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", dest="graph", action="store_false",
                    help="time K eager steps; by default the K timed steps are replays of one captured HIP graph "
                         "of a step (per-kernel durations always come from K eager steps before it)")
    ap.add_argument("--only", default="", help="comma list of gate,up,down (profiling aid)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 128 MiB read + 128 MiB write elementwise kernel three times, so that a "
                         "counter profile of this command holds a kernel of known traffic to scale by")
    ap.add_argument("--workload", choices=("mlp", "stack", "ppcx", "decode"), default="mlp",
                    help="mlp: the three MLP matrices of one layer (the headline); stack: every coded linear of "
                         "--layers layers resident at once, one pass at batch 64 (or --batch); ppcx: a predictive "
                         "frame against its dense reference, product with 96 rows (or --batch); decode: the "
                         "three MLP matrices decoded to dense BF16 (decode(), the fused store sink)")
    ap.add_argument("--layers", type=int, default=64)
    ap.add_argument("--no-groups", action="store_true",
                    help="one launch per linear instead of one for the matrices that take the same activations "
                         "(gate/up; in the stack also q/k/v)")
    ap.add_argument("--no-extras", action="store_true",
                    help="mlp at batch 1: leave out the batch-64 step and the whole-stack pass that the default run "
                         "adds to the line as `batch64` and `stack`")
    ap.add_argument("--no-stack", action="store_true", help="mlp at batch 1: leave out the whole-stack pass only")
    ap.add_argument("--distinct-layers", type=int, default=1,
                    help="stack: layers encoded from their own seeds; the rest are device copies of these")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this decode path runs on one GPU; --gpus must be 1 (no multi-GPU figure exists)")
    if args.workload == "mlp":
        args.batch = args.batch or 1  # the stack defaults to 64
    decode_only = args.workload == "decode"
    if decode_only:
        args.batch, args.no_groups = 0, True  # no activations: rows = 0 selects the store sink's tiling
    if args.workload == "ppcx":
        return run_predictive(args)
    if args.workload == "stack":
        if not 1 <= args.distinct_layers <= args.layers:
            sys.exit("bench.py: --distinct-layers must be between 1 and --layers")
        return run_stack(args)

    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    global GEMV_UP_TO
    GEMV_UP_TO = HipContextTensor.GEMV_UP_TO

    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a ROCm GPU")
    names = [s for s in args.only.split(",") if s] or list(SHAPES)
    tensors, frames, words_of = {}, {}, {}
    t_setup = time.perf_counter()
    for i, name in enumerate(SHAPES):
        if name not in names:
            continue
        rows, cols = SHAPES[name]
        w = synth_weights(i, rows, cols)
        t0 = time.perf_counter()
        frame = codec.encode(w)
        t1 = time.perf_counter()
        tensors[name] = HipContextTensor(frame, stride=1024, device="cuda:0",
                                         fused_segment=args.segment or None)
        t2 = time.perf_counter()
        if tensors[name].fused is None:
            sys.exit(f"bench.py: {name} is not eligible for the fused kernel: {tensors[name].fused_reason}")
        log(f"{name}: {rows}x{cols} mode {tensors[name].mode} frame {len(frame)} B "
            f"({8 * len(frame) / w.size:.3f} bit/weight) encode {t1 - t0:.1f}s index+upload {t2 - t1:.1f}s "
            f"resident mode {tensors[name].resident_mode} plan {tensors[name].fused_plan} "
            f"tiling {(tensors[name]._tiling(args.batch) if args.batch <= GEMV_UP_TO else tensors[name]._gemm_tiling())[3]}")
        frames[name] = frame
        words_of[name] = w
    log(f"setup {time.perf_counter() - t_setup:.1f}s")

    # the launches of a step: gate and up take the same activations and share one launch
    from georefine_amd.bitexact_context_gpu import HipLinearGroup
    pair = None
    if not args.no_groups and "gate" in names and "up" in names:
        pair = HipLinearGroup([tensors["gate"], tensors["up"]])

    # Device copies of the layer's matrices, taken in turn by the timed steps and launches, enough
    # that any one matrix's copies are twice the last-level cache: repeated passes over one 128 MB
    # matrix would find it in that cache, which a model of 64 layers never does.
    n_layers = max(1, -(-2 * LAST_LEVEL_CACHE_BYTES // min(tensors[n_].resident_bytes for n_ in names)))
    layers = [(tensors, pair)]
    for _ in range(n_layers - 1):
        copy_ = {n_: tensors[n_].clone() for n_ in names}
        layers.append((copy_, HipLinearGroup([copy_["gate"], copy_["up"]]) if pair is not None else None))
    log(f"{n_layers} device copies of the layer, taken in turn")

    def measure(m):
        """One workload at m activation rows (0: decode to dense): (result fields, x words)."""
        rng = np.random.default_rng(7)
        x_words = {k: bf16_words(rng.normal(0, 1, size=(max(m, 1), k))) for k in (5120, 17408)}
        x = {k: torch.from_numpy(v).view(torch.bfloat16).cuda() for k, v in x_words.items()}

        def units_of(tensors, pair):  # the launches of a step: (label, member names, callable)
            units = []
            if pair is not None and not decode_only:
                units.append(("gate+up", ["gate", "up"], lambda: pair.linear(x[5120])))
            for name in names:
                if decode_only:
                    units.append((name, [name], lambda name=name: tensors[name].decode(check=False)))
                elif not any(name in u[1] for u in units):
                    units.append((name, [name], lambda name=name: tensors[name].linear(x[SHAPES[name][1]])))
            return units

        per_layer = [units_of(*layer) for layer in layers]
        units = per_layer[0]
        if pair is not None and not decode_only:
            log(f"batch {m} gate+up: one launch, tiling {pair._tiling('waves' if m <= GEMV_UP_TO else 'gemm')[0][3]}")
        ms_per_step, per_kernel_ms, launch, timing = time_launches(
            torch, per_layer, args.steps, args.warmup, args.graph,
            lambda: sorted({n_ for ts, pr in layers for n_ in names if ts[n_].error.item()}
                           | {"gate+up" for ts, pr in layers if pr is not None and pr.error.item()}))
        if args.calibrate_copy:
            src = torch.ones(32 * 1024 * 1024, dtype=torch.int32, device="cuda")
            dst = torch.empty_like(src)
            for _ in range(3):
                torch.add(src, 1, out=dst)
            torch.cuda.synchronize()
        alg = {}
        for label, members, _ in units:
            parts = [algorithmic_bytes(tensors[n_], m) for n_ in members]
            alg[label] = {k: sum(p_[k] for p_ in parts) for k in parts[0]}
            if len(members) > 1:  # the members read one x
                alg[label]["total"] -= (len(members) - 1) * m * SHAPES[members[0]][1] * 2
            if decode_only:  # the dense matrix is written once
                alg[label]["total"] += sum(2 * SHAPES[n_][0] * SHAPES[n_][1] for n_ in members)
        step_bytes = sum(a_["total"] for a_ in alg.values())
        dense_bytes = sum(2 * SHAPES[n_][0] * SHAPES[n_][1] for n_ in names)
        value = step_bytes / (ms_per_step * 1e-3) / 1e9
        eff_bf16 = dense_bytes / (ms_per_step * 1e-3) / 1e9
        dom = max(per_kernel_ms, key=lambda n_: per_kernel_ms[n_])
        kernel = kernel_name(decode_only, m, "+" in dom, tensors[names[0]].fused_plan["seg_len"])
        traffic, traffic_source = recorded_traffic(decode_only, m, kernel)
        achieved = alg[dom]["total"] / (per_kernel_ms[dom] * 1e-3) / 1e9
        fields = {
            "value": round(value, 2), "ms_per_step": round(ms_per_step, 4),
            "config": {"workload": ("fused decode to dense BF16 (decode())" if decode_only else
                                    "fused decode-" + ("GEMV" if m <= GEMV_UP_TO else "GEMM") + ", batch %d" % m)
                                   + ", Qwen-27B-like MLP: gate/up 5120->17408, down 17408->5120, BCTX (16,4) frames"
                                   + (", residuals resident in packed 6-bit form"
                                      if any(tensors[n_].resident_mode != tensors[n_].mode for n_ in names) else ""),
                       "batch": m, "matrices": names, "launches": [u[0] for u in units],
                       "segment": tensors[names[0]].fused_plan["seg_len"], "launch": launch, "per_kernel_timing": timing,
                       "layer_copies": n_layers},
            "effective_bf16_GBps": round(eff_bf16, 2),
            "tok_s_equiv": round(eff_bf16 * 1e9 / MODEL_BF16_BYTES * m, 3) if m else None,
            "pct_hbm_roofline": round(100 * value / HBM_PEAK_GBPS, 2),
            "per_kernel": {n_: {"ms": round(per_kernel_ms[n_], 4), "alg_bytes": alg[n_]["total"],
                                "payload_bytes": alg[n_]["payload"], "index_bytes": alg[n_]["index"],
                                "table_bytes": alg[n_]["tables"],
                                "GBps": round(alg[n_]["total"] / (per_kernel_ms[n_] * 1e-3) / 1e9, 2),
                                "frac_of_hbm_peak": round(alg[n_]["total"] / (per_kernel_ms[n_] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
                           for n_ in per_kernel_ms},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                         "kernel": f"{kernel} on {dom}"},
        }
        if m > GEMV_UP_TO:
            # the matrix cores' share: useful flops of the dominant launch against the dense BF16 peak
            flops = sum(2.0 * m * SHAPES[n_][0] * SHAPES[n_][1] for n_ in dom.split("+"))
            fields["mfma"] = {"achieved": round(flops / (per_kernel_ms[dom] * 1e-3) / 1e12, 2), "peak": 2500.0,
                              "unit": "TFLOP/s", "frac": round(flops / (per_kernel_ms[dom] * 1e-3) / 2.5e15, 4)}
        return fields, x_words

    fields, x_words = measure(args.batch)
    result = {
        "metric": "compressed-weight decode GB/s (coded bytes read + dense BF16 written)" if decode_only
                  else "compressed-weight decode-GEMV GB/s",
        "value": fields.pop("value"), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": fields.pop("ms_per_step"), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u32 rANS state / bf16 weights / fp32 accumulate", "data": "synthetic",
    }
    result.update(fields)
    copy_rate = measured_copy_gbps(torch)
    result["hbm_copy_measured_GBps"] = round(copy_rate, 1)
    result["pct_of_measured_copy"] = round(100 * result["value"] / copy_rate, 2)
    headline = args.workload == "mlp" and args.batch == 1 and not args.only and not args.no_extras
    if headline:
        # the other two figures of the metric, timed in the same run: the MLP step at batch 64
        # (fused GEMM on the matrix cores) and one pass through a whole resident stack
        log("batch 64 ...")
        b64, _ = measure(64)
        b64.pop("config")
        result["batch64"] = b64
    if not args.no_cpu_baseline:
        log("timing the CPU oracle on whole frames ...")
        result["cpu_baseline"] = cpu_baseline(frames, words_of, x_words)
        result["cpu_baseline"]["host"] = host_description()
    if headline and not args.no_stack:
        del tensors, pair, layers
        torch.cuda.empty_cache()
        log("whole stack ...")
        stack_args = argparse.Namespace(**vars(args))
        stack_args.batch, stack_args.steps, stack_args.warmup = 64, max(3, args.steps // 10), max(2, args.warmup // 10)
        result["stack"] = run_stack(stack_args, as_dict=True)
    print(json.dumps(result), flush=True)


def kernel_name(decode_only, m, grouped, seg_len):
    """The kernel a launch of the workload runs (as rocprofv3 names it)."""
    ahead = "true" if seg_len == 64 else "false"  # 64-symbol segments: the walker that reads a segment's residuals once
    if decode_only:
        return f"grf::fused_walk_kernel<grf::SegmentWalkT<{ahead}>, 1, 1>"
    # (last template argument 1: the scan for frames without whole-range contexts, which these are)
    if m <= GEMV_UP_TO:
        rows = min(m, 2)  # the wave-unit GEMV carries at most two rows per launch
        return (f"grf::fused_wave_group_kernel<grf::SegmentWalkT<false>, {rows}, 1>" if grouped
                else f"grf::fused_wave_kernel<grf::SegmentWalkT<false>, {rows}, 1>")
    return ("grf::fused_gemm_group_kernel<grf::SegmentWalkT<false>, MT, 1>" if grouped
            else "grf::fused_gemm_kernel<grf::SegmentWalkT<false>, MT, 1>")


def kernel_sources_sha256():
    """Digest of the device sources: a recorded counter figure is only quoted for these."""
    import hashlib
    h = hashlib.sha256()
    for path in sorted((ROOT / "georefine_amd" / "csrc").glob("*")):
        if path.suffix in (".h", ".hip"):
            h.update(path.name.encode() + b"\0" + path.read_bytes())
    return h.hexdigest()


def recorded_traffic(decode_only, m, kernel):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE
    record (bench.py cannot read hardware counters itself), and where the figure comes from.
    The record names the kernels it measured and the digest of the device sources it was taken
    with; for another kernel or other sources the figure is withheld (None) and the reason given."""
    name = ("fused_store_decode_qwen27b_mlp_traffic.json" if decode_only else
            "fused_gemv_m1_qwen27b_mlp_traffic.json" if m == 1 else
            "fused_gemm_m64_qwen27b_mlp_traffic.json" if m == 64 else None)
    if name is None or not (ROOT / "profiles" / name).exists():
        return None, "no counter record for this workload"
    record = json.loads((ROOT / "profiles" / name).read_text())
    per_kernel = record.get("traffic_bytes_per_launch")
    short = kernel.split("<")[0].split("::")[-1]
    if not isinstance(per_kernel, dict) or short not in per_kernel:
        return None, f"profiles/{name} holds no figure for {short}"
    if record.get("kernel_sources_sha256") != kernel_sources_sha256():
        return None, f"profiles/{name} was recorded with other kernel sources (its figure for {short}: {per_kernel[short]:.0f} B)"
    return per_kernel[short], f"recorded: profiles/{name} (rocprofv3 --pmc, same kernel sources)"


def time_launches(torch, per_layer, steps, warmup, graph, errors):
    """(ms per step, {label: ms per launch}, how the step was launched, how launches were timed).

    `per_layer[c]` holds the launches of a step on copy c of the layer's matrices; step i runs
    on copy i mod len(per_layer), so no step finds its matrices in the caches.  After `warmup`
    eager steps: each launch is captured twelve times into a HIP graph of its own, over the
    copies in turn, and the replays are bracketed by events on the launch stream, which gives
    the kernel's duration without the host's per-launch latency (eager events around single
    launches where capture is not possible or --no-graph is given); then exactly `steps` steps,
    replayed from graphs of up to 96 consecutive steps, are timed on the host clock between
    synchronisations."""
    copies = len(per_layer)

    def step(i):
        return [run() for _, _, run in per_layer[i % copies]]

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    bad = errors()
    if bad:
        sys.exit(f"bench.py: decoder error word set for {bad}")
    per_kernel_ms = {}
    timing = f"HIP events around 12 launches per graph replay, over {copies} device copies of the matrices in turn"
    if graph:
        try:
            for j, (label, _, _) in enumerate(per_layer[0]):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    for i in range(12):
                        per_layer[i % copies][j][2]()
                g.replay()
                torch.cuda.synchronize()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                replays = max(2, steps // 10)
                a.record()
                for _ in range(replays):
                    g.replay()
                b.record()
                torch.cuda.synchronize()
                per_kernel_ms[label] = a.elapsed_time(b) / (12 * replays)
        except Exception as exc:
            log(f"graph capture failed ({exc}); timing eager launches")
            per_kernel_ms = {}
    if not per_kernel_ms:
        timing = "HIP events around single eager launches"
        n_units = len(per_layer[0])
        starts = [[torch.cuda.Event(enable_timing=True) for _ in range(n_units)] for _ in range(steps)]
        ends = [[torch.cuda.Event(enable_timing=True) for _ in range(n_units)] for _ in range(steps)]
        torch.cuda.synchronize()
        for s_ in range(steps):
            for j, (_, _, run) in enumerate(per_layer[s_ % copies]):
                starts[s_][j].record()
                run()
                ends[s_][j].record()
        torch.cuda.synchronize()
        per_kernel_ms = {label: float(np.mean([starts[s_][j].elapsed_time(ends[s_][j]) for s_ in range(steps)]))
                         for j, (label, _, _) in enumerate(per_layer[0])}
    launch = "eager"
    wall = None
    if graph:
        # consecutive steps captured once and replayed: the launches are submitted together, which
        # takes the host's per-launch latency out of the gaps between kernels
        try:
            chunk = min(steps, 96) // copies * copies or steps  # whole turns through the copies
            plan = [(chunk, steps // chunk)] + ([(steps % chunk, 1)] if steps % chunk else [])
            graphs = []
            for length, times in plan:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    for i in range(length):
                        step(i)
                g.replay()
                graphs.append((g, times))
            torch.cuda.synchronize()
        except Exception as exc:  # keep the eager figure
            log(f"graph capture failed ({exc}); reporting the eager steps")
        else:
            wall0 = time.perf_counter()
            for g, times in graphs:
                for _ in range(times):
                    g.replay()
            torch.cuda.synchronize()
            wall = time.perf_counter() - wall0
            launch = "hip graph replay"
    if wall is None:
        torch.cuda.synchronize()
        wall0 = time.perf_counter()
        for i in range(steps):
            step(i)
        torch.cuda.synchronize()
        wall = time.perf_counter() - wall0
    bad = errors()
    if bad:
        sys.exit(f"bench.py: decoder error word set for {bad}")
    return wall / steps * 1e3, per_kernel_ms, launch, timing


if __name__ == "__main__":
    main()

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

The K timed steps are replays of HIP graphs of consecutive steps (--no-graph times eager
steps instead); the per-launch durations come from device timestamps inside a graph of the
same steps.  The default run adds the other configurations of the metric to the same line:
`m_invariant_policy` (the down projection at 1 and 6 rows under the batch-invariant route, beside
the default route), `batch64` (the MLP step at batch 64, fused GEMM), `attention` (q/k/v/o at batch 1..128 through
the batch-invariant GEMM), `ppcx` (a predictive frame, products with 1 and 96 rows) and `stack`
(every coded linear of a 64-layer model resident at once, one pass at batch 64).
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


def synth_weights_f32(seed, rows, cols):
    """The same distribution drawn in float32 (twice as fast; other values than synth_weights
    gives for a seed): for the whole-stack workload, whose set-up is mostly this."""
    rng = np.random.default_rng(seed)
    out = np.empty((rows, cols), dtype=np.uint16)
    scale = rng.lognormal(0.0, 0.5, size=(rows, 1)).astype(np.float32) * np.float32(0.02)
    step = 4096
    for lo in range(0, rows, step):
        hi = min(rows, lo + step)
        w = rng.standard_normal(size=(hi - lo, cols), dtype=np.float32) * scale[lo:hi]
        mask = rng.random((hi - lo, cols), dtype=np.float32) < np.float32(1e-3)
        w = np.where(mask, w * np.float32(10.0), w)
        out[lo:hi] = bf16_words(w)
    return out


GEMV_UP_TO = 2  # rows linear() gives to the vector-ALU kernel; read from HipContextTensor once it is imported


def algorithmic_bytes(t, m, gemm=None):
    """Bytes one fused GEMV / GEMM launch has to touch once: both streams, the fused index,
    the per-class lookup tables, labels, activations and outputs.  ``gemm``: the launch runs
    the matrix-core kernel (default: from the row count, as linear() routes)."""
    b = t.buffers
    n = lambda k: b[k].numel() * b[k].element_size()
    rows, cols = t.shape
    # (the resident residual array starts every row class on a multiple of 16 rows: the rows it
    # holds beyond the matrix's are never read and are not counted)
    payload = t._main_bytes + min(n("residual_stream"), rows * cols * 3 // 4)
    if gemm is None:
        gemm = m > GEMV_UP_TO
    _, tile_rows, tile_class, _ = t._gemm_tiling() if gemm else t._tiling(m)
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


def calibration_copy(torch):
    """A plain 128 MiB read + 128 MiB write elementwise kernel, three times: a kernel of known
    traffic for a counter profile of this command to scale its FETCH_SIZE / WRITE_SIZE by."""
    src = torch.ones(32 * 1024 * 1024, dtype=torch.int32, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(3):
        torch.add(src, 1, out=dst)
    torch.cuda.synchronize()


def launch_fields(alg_total, ms):
    gbps = alg_total / (ms * 1e-3) / 1e9
    return {"ms": round(ms, 4), "alg_bytes": int(alg_total), "GBps": round(gbps, 2),
            "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4)}


def roofline_fields(alg_total, ms, kernel, traffic=None, traffic_source=None):
    gbps = alg_total / (ms * 1e-3) / 1e9
    out = {"bound": "hbm", "achieved": round(gbps, 2), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
           "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": traffic, "kernel": kernel}
    if traffic_source:
        out["traffic_source"] = traffic_source
    return out


ATTENTION = {"q": (6144, 5120), "k": (1024, 5120), "v": (1024, 5120), "o": (5120, 6144)}
ATTENTION_BATCHES = (1, 8, 32, 64, 128)


def run_attention(args, as_dict=False):
    """The attention projections -- q 5120->6144, k/v 5120->1024, o 6144->5120 -- at batch 1, 8,
    32, 64 and 128 through the batch-invariant route: every row count runs the matrix-core GEMM
    (q, k and v, which take the same rows, in one launch), and a row's output bits are checked
    to be the same at every batch.  The batch-1 time of the default route (the VALU GEMV, whose
    rows are bit-equal among themselves only) is reported beside it."""
    import torch
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor, HipLinearGroup
    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a ROCm GPU")
    t0 = time.perf_counter()
    base = {}
    for i, (name, (rows, cols)) in enumerate(ATTENTION.items()):
        # q, k and v share a launch, so they are indexed at one segment length
        base[name] = HipContextTensor(codec.encode(synth_weights(10 + i, rows, cols)), stride=1024, device="cuda:0",
                                      fused_segment=64)
        if base[name].fused is None:
            sys.exit(f"bench.py: {name} is not eligible for the fused kernels: {base[name].fused_reason}")
    resident = sum(t.resident_bytes for t in base.values())
    copies = max(1, -(-2 * LAST_LEVEL_CACHE_BYTES // resident))
    sets = [base] + [{k: v.clone() for k, v in base.items()} for _ in range(copies - 1)]
    groups = [HipLinearGroup([s_["q"], s_["k"], s_["v"]]) for s_ in sets]
    log(f"attention: 4 matrices coded and resident in {time.perf_counter() - t0:.1f}s, {copies} device copies in turn")
    rng = np.random.default_rng(7)
    x = {k: torch.from_numpy(bf16_words(rng.normal(0, 1, size=(128, k)))).view(torch.bfloat16).cuda() for k in (5120, 6144)}
    steps, warmup = max(10, args.steps // 2), max(4, args.warmup // 4)

    def errors():
        return sorted({n_ for s_ in sets for n_, t in s_.items() if t.error.item()}
                      | {"q+k+v" for g in groups if g.error.item()})

    def per_layer(m, invariant):
        return [[("q+k+v", ["q", "k", "v"], lambda g=g: g.linear(x[5120][:m], batch_invariant=invariant)),
                 ("o", ["o"], lambda t=s_["o"]: t.linear(x[6144][:m], batch_invariant=invariant))]
                for s_, g in zip(sets, groups)]

    def alg_of(m, gemm):
        parts = {n_: algorithmic_bytes(base[n_], m, gemm=gemm)["total"] for n_ in ATTENTION}
        return {"q+k+v": parts["q"] + parts["k"] + parts["v"] - 2 * m * 5120 * 2, "o": parts["o"]}

    def one(m, invariant):
        ms_step, per_ms, launch, timing, clocks = time_launches(torch, per_layer(m, invariant), steps, warmup,
                                                                args.graph, errors)
        alg = alg_of(m, invariant or m > GEMV_UP_TO)
        dom = max(alg, key=lambda k: alg[k])
        gemm = invariant or m > GEMV_UP_TO
        kernel = ("grf::fused_gemm_group_kernel / fused_gemm_wide_group_kernel<grf::SegmentWalkT<false>, MT, 1>" if gemm
                  else f"grf::fused_wave_group_kernel<grf::SegmentWalkT<false>, {min(m, 2)}, 1>")
        total = sum(alg.values())
        return {"ms_per_pass": round(ms_step, 4), "GBps": round(total / (ms_step * 1e-3) / 1e9, 2), "launch": launch,
                "rows_per_s": round(m / (ms_step * 1e-3), 1), **clocks,
                "per_kernel": {k: launch_fields(alg[k], per_ms[k]) for k in per_ms},
                "roofline": roofline_fields(alg[dom], per_ms[dom], f"{kernel} on {dom}")}, timing

    # a row's bits do not depend on the batch it arrives in: rows of every batch against batch 128
    full = [groups[0].linear(x[5120], batch_invariant=True, check=True), base["o"].linear(x[6144], batch_invariant=True,
                                                                                          check=True)]
    equal = True
    for m in ATTENTION_BATCHES:
        ys = groups[0].linear(x[5120][:m], batch_invariant=True) + [base["o"].linear(x[6144][:m], batch_invariant=True)]
        want = list(full[0]) + [full[1]]
        equal = equal and all(torch.equal(y.view(torch.uint16), w[:m].view(torch.uint16)) for y, w in zip(ys, want))
    if not equal:
        sys.exit("bench.py: attention rows differ between batches on the batch-invariant route")
    batches, timing = {}, ""
    for m in ATTENTION_BATCHES:
        batches[str(m)], timing = one(m, True)
        log(f"attention batch {m}: {batches[str(m)]['ms_per_pass']} ms per pass")
    default1, _ = one(1, False)
    if args.calibrate_copy:
        calibration_copy(torch)
    result = {
        "config": {"workload": "attention projections q 5120->6144, k/v 5120->1024, o 6144->5120 (BCTX (16,4) frames), "
                               "q/k/v in one launch, o in another; every batch through the matrix-core GEMM "
                               "(batch-invariant route)",
                   "batches": list(ATTENTION_BATCHES), "steps": steps, "warmup": warmup, "layer_copies": copies,
                   "per_kernel_timing": timing},
        "coded_resident_bytes": resident, "dense_bf16_bytes": sum(2 * r * c for r, c in ATTENTION.values()),
        "rows_bit_equal_across_batches": bool(equal),
        "batch_invariant": batches,
        "default_route_batch1": default1,
    }
    sets.clear()
    groups.clear()
    base.clear()
    torch.cuda.empty_cache()
    if as_dict:
        return result
    print(json.dumps({"metric": "compressed-weight decode-GEMV GB/s", "value": batches["1"]["GBps"], "unit": "GB/s",
                      "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": batches["1"]["ms_per_pass"],
                      "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
                      "dtype": "u32 rANS state / bf16 weights / fp32 accumulate", "data": "synthetic", **result}), flush=True)


PPCX_BATCHES = (1, 96)


def run_predictive(args, as_dict=False):
    """A 5120 x 17408 target coded (PPCX) against a reference that is the target plus N(0, 0.002)
    noise, as a loaded model serves it: the tensor keeps the 4-bit context plane of its
    reference from load on, so no reference is resident or decoded.  One step = the product of
    the coded target with the activation rows, on three resident copies in turn: one row (the
    fused GEMV) and 96 rows = 16 users x (5 draft tokens + 1), the verify shape (activations
    packed, then the fused GEMM); --batch picks a single row count."""
    import torch
    from georefine_amd import bitexact_predictive_codec as ppcx
    from georefine_amd.bitexact_predictive_gpu import HipPredictiveTensor

    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a ROCm GPU")
    batches = (args.batch,) if args.batch and not as_dict else PPCX_BATCHES
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
    log(f"PPCX frame {len(frame)} B ({8 * len(frame) / target.size:.3f} bit/weight) mode {t.mode}; setup {time.perf_counter() - t0:.1f}s; "
        f"rows per label {np.bincount(t.buffers['labels'].cpu().numpy(), minlength=16).tolist()}; GEMV tiling "
        f"{t._tiling_for('waves')[3]}; GEMM tiling {t._tiling_for('gemm')[3]}")
    copies = [t, t.clone(), t.clone()]  # three targets in rotation: more bytes than the caches hold
    steps, warmup = (args.steps, args.warmup) if not as_dict else (max(10, args.steps // 2), max(4, args.warmup // 4))
    x_all = torch.from_numpy(bf16_words(np.random.default_rng(7).normal(0, 1, size=(max(batches), cols)))).view(torch.bfloat16).cuda()
    dense = torch.from_numpy(target).view(torch.bfloat16).cuda().float()
    for m in batches:
        want = torch.nn.functional.linear(x_all[:m].float(), dense)
        scale = torch.nn.functional.linear(x_all[:m].float().abs(), dense.abs())
        got = t.linear(None, x_all[:m], check=True).float()
        if not bool((got - want).abs().le(1e-2 * want.abs().clamp_min(1e-3 * scale)).all()):
            sys.exit(f"bench.py: the fused product with {m} rows is outside 1e-2 of the dense product")
    del dense, want, scale, got
    coded = t.resident_bytes
    out = {}
    for m in batches:
        x = x_all[:m]
        per_layer = [[("product", ["target"], lambda c=c: c.linear(None, x))] for c in copies]
        ms_step, per_ms, launch, timing, clocks = time_launches(
            torch, per_layer, steps, warmup, args.graph, lambda: ["target"] if any(c.error.item() for c in copies) else [])
        # bytes one product has to touch once: everything the tensor keeps on the device (the coded
        # target, its index and tables, the 4-bit context plane of the reference), activations, outputs
        alg = coded + m * cols * 2 + m * rows * 2
        kernel = ("grf::fused_wave_kernel<PpcxWalk, 1, SCAN>" if m == 1 else
                  "pack_activations_kernel + grf::fused_gemm_kernel / fused_gemm_wide_kernel<PpcxWalk, MT, SCAN> (+ gemm_sum_parts_kernel)")
        traffic, source = recorded_traffic(False, m, kernel, prefix="ppcx")
        out[str(m)] = {"ms_per_product": round(ms_step, 4), "launch": launch, "per_kernel_timing": timing, **clocks,
                       "GBps": round(alg / (ms_step * 1e-3) / 1e9, 2), "rows_per_s": round(m / (ms_step * 1e-3), 1),
                       "algorithmic_bytes_per_product": alg,
                       "roofline": roofline_fields(alg, per_ms["product"], kernel + " (all launches of a product)", traffic, source)}
        log(f"ppcx batch {m}: {ms_step:.4f} ms per product")
    if args.calibrate_copy:
        calibration_copy(torch)
    n = target.size
    result = {
        "config": {"workload": "PPCX target 5120x17408 coded against a reference (target + N(0, 0.002)), products as "
                               "served: contexts of the reference resident as a 4-bit plane, no dense reference; three "
                               "resident copies in turn", "batches": list(batches), "steps": steps, "warmup": warmup},
        "frame_bytes": len(frame), "frame_bits_per_weight": round(8 * len(frame) / n, 3),
        "resident_bytes": coded, "resident_bits_per_weight": round(8 * coded / n, 3),
        "context_plane_bytes": n // 2, "frame_mode": t.mode, "resident_mode": t.resident_mode,
        "batch": out,
    }
    copies.clear()
    del t
    torch.cuda.empty_cache()
    if as_dict:
        return result
    first = out[str(batches[-1])]
    print(json.dumps({"metric": "compressed-weight decode-GEMV GB/s", "value": first["GBps"], "unit": "GB/s", "n_gpus": 1,
                      "steps": steps, "warmup": warmup, "ms_per_step": first["ms_per_product"], "higher_is_better": True,
                      "scaling": "weak", "vs_baseline": None, "dtype": "u32 rANS state / bf16 weights / fp32 accumulate",
                      "data": "synthetic", **result, "roofline": first["roofline"]}), flush=True)


# The whole-stack workload.  "qwen": the linear shapes of the 27B model the reference serves
# (GCR/bitexact_context_mtp.py:244-260 and the reference's kernel tuning tables): 16 full-attention
# layers, 48 linear-attention layers, the vocabulary matrix twice (embedding and head).
# "baseline": 64 layers of the attention and MLP shapes the other workloads use.
MLP3 = {"gate": (17408, 5120), "up": (17408, 5120), "down": (5120, 17408)}
STACKS = {
    "qwen": {"attn": dict({"q": (12288, 5120), "k": (1024, 5120), "v": (1024, 5120), "o": (5120, 6144)}, **MLP3),
             "gdn": dict({"in_proj": (16480, 5120), "out_proj": (5120, 6144)}, **MLP3),
             "vocab": (248320, 5120), "attn_every": 4},
    "baseline": {"attn": dict(LAYER), "gdn": None, "vocab": None, "attn_every": 1},
}
SHARED_INPUT = (("q", "k", "v"), ("gate", "up"))  # siblings that take the same rows: one launch each


def stack_job(job):
    """Worker process: one matrix drawn, encoded, validated, indexed and laid out for the kernels
    (HipContextTensor.host_prepare needs no GPU); the result goes to a file."""
    import pickle
    from georefine_amd import bitexact_context_codec as codec
    from georefine_amd.bitexact_context_gpu import HipContextTensor
    key, seed, (rows, cols), residual, folder = job
    frame = codec.encode(synth_weights_f32(seed, rows, cols), residual=residual)
    # (blocks of sixteen rows: the pass runs the matrix-core kernel)
    prepared = HipContextTensor.host_prepare(frame, stride=1024, fused_segment=64, residual_block=16)
    path = os.path.join(folder, "_".join(map(str, key)) + ".pickle")
    with open(path, "wb") as f:
        pickle.dump((len(frame), prepared), f, protocol=pickle.HIGHEST_PROTOCOL)
    return key, path


class StackPrep:
    """Host half of the whole-stack workload in worker processes: every distinct matrix is drawn,
    encoded, validated, indexed and laid out for the kernels; the device objects are
    constructed later from the results, by the process that owns the GPU.  Started before that
    process touches the GPU (the workers are forked, and never touch it), it runs beside the
    other workloads' GPU phases.  Processes, not threads: a busy thread would hold the
    interpreter's lock for milliseconds at a time, which the timed regions of the other
    workloads, themselves a few milliseconds long, cannot afford."""

    def __init__(self, args):
        import atexit
        import multiprocessing
        import shutil
        import tempfile
        from concurrent.futures import ProcessPoolExecutor
        spec = STACKS[args.stack_shapes]
        self.spec, self.t0 = spec, time.perf_counter()
        kinds = [k for k in ("attn", "gdn") if spec[k]]
        n_attn = sum(1 for i in range(args.layers) if spec["gdn"] is None or i % spec["attn_every"] == spec["attn_every"] - 1)
        self.counts = {"attn": n_attn, "gdn": args.layers - n_attn}
        self.distinct = {k: max(1, min(args.distinct_layers, self.counts[k])) for k in kinds if self.counts[k]}
        self.folder = tempfile.mkdtemp(prefix="georefine_bench_", dir="/dev/shm" if os.path.isdir("/dev/shm") else None)
        atexit.register(shutil.rmtree, self.folder, ignore_errors=True)
        jobs = []
        if spec["vocab"]:
            jobs.append((("vocab", 0, "vocab"), 7777, spec["vocab"], "raw6", self.folder))  # the longest job first
        for kind, count in self.distinct.items():
            for d in range(count):
                for j, (name, shape) in enumerate(spec[kind].items()):
                    jobs.append(((kind, d, name), 100000 * (1 + kinds.index(kind)) + 100 * d + j, shape, "auto", self.folder))
        # (the box's share of host cores is 16 whatever it reports; half of them)
        self.pool = ProcessPoolExecutor(max_workers=max(1, min(8, (os.cpu_count() or 2) // 2)),
                                        mp_context=multiprocessing.get_context("fork"))
        self.futures = [self.pool.submit(stack_job, job) for job in jobs]
        self.done = None

    def results(self):
        """{key: (frame bytes, prepared)}; waits for the workers."""
        import pickle
        if self.done is None:
            paths = dict(f.result() for f in self.futures)
            self.pool.shutdown()
            log(f"stack: {len(paths)} distinct matrices drawn, encoded and indexed {time.perf_counter() - self.t0:.1f}s "
                f"after the start")
            self.done = paths
        out = {}
        for key, path in self.done.items():
            with open(path, "rb") as f:
                out[key] = pickle.load(f)
            os.unlink(path)
        return out

    def wait(self):
        if self.done is None:
            self.done = dict(f.result() for f in self.futures)
            self.pool.shutdown()
            log(f"stack: {len(self.done)} distinct matrices drawn, encoded and indexed {time.perf_counter() - self.t0:.1f}s "
                f"after the start")


def run_stack(args, as_dict=False, prep=None):
    """Every coded linear of a 64-layer model resident at once, one pass at batch 64: a row
    gather from the embedding matrix, every layer's projections (siblings that take the same
    rows share a launch), the head.  `--distinct-layers` layers of each kind are drawn and
    encoded from their own seeds; the others are device copies of those in rotation (their own
    buffers, so a pass streams every layer's bytes from HBM, but no further host encoding)."""
    prep = prep or StackPrep(args)  # (forks its workers: before this process touches the GPU)
    import torch
    from georefine_amd.bitexact_context_gpu import HipContextTensor, HipLinearGroup
    global GEMV_UP_TO
    GEMV_UP_TO = HipContextTensor.GEMV_UP_TO

    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a ROCm GPU")
    m = args.batch or 64
    spec = prep.spec
    done = prep.results()
    t0 = time.perf_counter()
    base, frame_len = {}, {}
    for key, (frame_bytes, prepared) in done.items():
        t = HipContextTensor(b"", stride=1024, device="cuda:0", prepared=prepared)
        if t.fused is None:
            sys.exit(f"bench.py: {key} is not eligible for the fused kernels: {t.fused_reason}")
        base[key], frame_len[key] = t, frame_bytes
    done.clear()
    log(f"stack: uploaded in {time.perf_counter() - t0:.1f}s")
    gemm = m > GEMV_UP_TO
    layers, used = [], {k: 0 for k in prep.distinct}
    for i in range(args.layers):
        kind = "attn" if spec["gdn"] is None or i % spec["attn_every"] == spec["attn_every"] - 1 else "gdn"
        d = used[kind] % prep.distinct[kind]
        first = used[kind] < prep.distinct[kind]
        used[kind] += 1
        src = {name: base[(kind, d, name)] for name in spec[kind]}
        layers.append((kind, src if first else {k: v.clone() for k, v in src.items()}))
    vocab = None
    if spec["vocab"]:
        head = base[("vocab", 0, "vocab")]
        vocab = {"embedding": head.clone(), "head": head}
    everything = [t for _, layer in layers for t in layer.values()] + (list(vocab.values()) if vocab else [])
    for t in everything:
        t._gemm_tiling() if gemm else t._tiling(m)
    torch.cuda.synchronize()
    frame_bytes = 0
    # frame bytes of the whole stack: every layer's frames (copies are the same frames again)
    seen = {k: 0 for k in prep.distinct}
    for kind, _ in layers:
        d = seen[kind] % prep.distinct[kind]
        seen[kind] += 1
        frame_bytes += sum(frame_len[(kind, d, name)] for name in spec[kind])
    if vocab:
        frame_bytes += 2 * frame_len[("vocab", 0, "vocab")]
    resident = sum(t.resident_bytes for t in everything)
    dense = sum(2 * t.shape[0] * t.shape[1] for t in everything)
    log(f"{args.layers} layers resident: {dense} BF16 bytes as {frame_bytes} frame bytes, {resident} device bytes; "
        f"torch reports {torch.cuda.memory_allocated()} allocated")

    rng = np.random.default_rng(7)
    widths = {t.shape[1] for t in everything}
    x = {k: torch.from_numpy(bf16_words(rng.normal(0, 1, size=(m, k)))).view(torch.bfloat16).cuda() for k in widths}
    ids = torch.from_numpy(rng.integers(0, spec["vocab"][0], size=m)).cuda() if vocab else None

    grouped = not args.no_groups
    launches = []  # (label, members as tensors, callable) of one pass
    if vocab:
        launches.append(("embedding", [], lambda t=vocab["embedding"]: t.gather_rows(ids, check=False, validate=False)))
    for kind, layer in layers:
        rest = list(layer)
        for sib in SHARED_INPUT:
            if grouped and all(n_ in layer for n_ in sib):
                g = HipLinearGroup([layer[n_] for n_ in sib])
                launches.append(("+".join(sib), [layer[n_] for n_ in sib],
                                 lambda g=g, w=layer[sib[0]].shape[1]: g.linear(x[w], batch_invariant=gemm)))
                rest = [n_ for n_ in rest if n_ not in sib]
        for name in rest:
            launches.append((name, [layer[name]], lambda t=layer[name]: t.linear(x[t.shape[1]], batch_invariant=gemm)))
    if vocab:
        launches.append(("head", [vocab["head"]], lambda t=vocab["head"]: t.linear(x[t.shape[1]], batch_invariant=gemm)))
    # (a pass in model order: the order above is by layer, siblings first -- every launch reads its own bytes,
    # so the order changes nothing that is measured)
    torch.cuda.synchronize()

    ms_per_step, per_ms, launch, timing, clocks = time_launches(
        torch, [launches], args.steps, args.warmup, args.graph,
        lambda: sorted({label for label, members, _ in launches for t in members if t.error.item()}))
    alg, count = {}, {}
    for label, members, _ in launches:
        if label == "embedding":  # the rows gathered: their share of both streams, written dense
            t = vocab["embedding"]
            total = int(m * (algorithmic_bytes(t, 0, gemm=False)["payload"] / t.shape[0] + 2 * t.shape[1]))
        else:
            total = sum(algorithmic_bytes(t, m, gemm=gemm)["total"] for t in members) - (len(members) - 1) * m * members[0].shape[1] * 2
        alg[label] = alg.get(label, 0) + total
        count[label] = count.get(label, 0) + 1
    step_bytes = sum(alg.values())
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    share = {label: per_ms[label] * count[label] for label in per_ms}  # ms of a pass spent in each kind of launch
    dom = max((l_ for l_ in alg if l_ != "embedding"), key=lambda l_: alg[l_])  # the kind that moves most bytes
    kernel = ("grf::fused_gemm_group_kernel<grf::SegmentWalkT<false>, MT, 1>" if "+" in dom else
              "grf::fused_gemm_kernel<grf::SegmentWalkT<false>, MT, 1>") if gemm else kernel_name(False, m, "+" in dom, 64)
    shapes_text = "; ".join(f"{k}: " + ", ".join(f"{n_} {c}->{r}" for n_, (r, c) in spec[k].items())
                            for k in ("attn", "gdn") if spec[k])
    result = {
        "metric": "compressed-weight decode-GEMV GB/s", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u32 rANS state / bf16 weights / fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": f"whole stack resident: {args.layers} layers ({prep.counts['attn']} attention, "
                               f"{prep.counts['gdn']} linear-attention; {shapes_text})"
                               + (f", embedding and head {spec['vocab'][0]}x{spec['vocab'][1]}" if vocab else "")
                               + f"; one pass through every coded linear at batch {m} (the embedding: a gather of "
                                 f"{m} rows); {dense / 1e9:.1f} GB of dense BF16 held as {frame_bytes / 1e9:.1f} GB of frames",
                   "shapes": args.stack_shapes, "batch": m, "layers": args.layers,
                   "distinct_layers": dict(prep.distinct), "linears": len(everything), "launches_per_pass": len(launches),
                   "launch": launch, "launches": "siblings that take the same rows share a launch" if grouped else "one per linear",
                   "per_kernel_timing": timing,
                   "vocabulary_frame": "mode 0 (packed 6-bit residuals written directly); the embedding is a device "
                                       "copy of the head's frame" if vocab else None},
        "dense_bf16_bytes": dense, "frame_bytes": frame_bytes, "resident_device_bytes": resident,
        "algorithmic_bytes_per_step": step_bytes,
        "effective_bf16_GBps": round(dense / (ms_per_step * 1e-3) / 1e9, 2),
        "tok_s_equiv": round(m / (ms_per_step * 1e-3), 1),
        "pct_hbm_roofline": round(100 * value / HBM_PEAK_GBPS, 2), **clocks,
        "per_kernel": {l_: dict(launch_fields(alg[l_] / count[l_], per_ms[l_]), launches=count[l_],
                                ms_of_pass=round(share[l_], 3)) for l_ in per_ms},
        "roofline": roofline_fields(alg[dom] / count[dom], per_ms[dom], f"{kernel} on {dom} ({count[dom]} launches per pass)"),
    }
    if as_dict:  # as a key of the headline line: the fields that line carries itself are left out
        for key in ("metric", "unit", "n_gpus", "higher_is_better", "scaling", "vs_baseline", "dtype", "data"):
            result.pop(key)
    launches.clear()
    layers.clear()
    base.clear()
    everything.clear()
    vocab = None
    torch.cuda.empty_cache()
    if as_dict:
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
    ap.add_argument("--residual-block", type=int, default=0,
                    help="mlp: rows per block of the resident residual order (0 = by batch: 16 above 2 rows, else the GEMV unit's)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", dest="graph", action="store_false",
                    help="time K eager steps; by default the K timed steps are replays of one captured HIP graph "
                         "of a step (per-kernel durations always come from K eager steps before it)")
    ap.add_argument("--only", default="", help="comma list of gate,up,down (profiling aid)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 128 MiB read + 128 MiB write elementwise kernel three times, so that a "
                         "counter profile of this command holds a kernel of known traffic to scale by")
    ap.add_argument("--workload", choices=("mlp", "stack", "ppcx", "decode", "attention"), default="mlp",
                    help="mlp: the three MLP matrices of one layer (the headline); stack: every coded linear of "
                         "--layers layers resident at once, one pass at batch 64 (or --batch); ppcx: a predictive "
                         "frame as served, products with 1 and 96 rows (or --batch); attention: q/k/v/o at batch "
                         "1..128 through the batch-invariant GEMM; decode: the three MLP matrices decoded to dense "
                         "BF16 (decode(), the fused store sink)")
    ap.add_argument("--stack-shapes", choices=tuple(STACKS), default="qwen",
                    help="stack: qwen = the linear shapes of the 27B model (16 attention and 48 linear-attention "
                         "layers, embedding and head); baseline = 64 layers of q/k/v/o/gate/up/down")
    ap.add_argument("--layers", type=int, default=64)
    ap.add_argument("--no-groups", action="store_true",
                    help="one launch per linear instead of one for the matrices that take the same activations "
                         "(gate/up; in the stack also q/k/v)")
    ap.add_argument("--no-extras", action="store_true",
                    help="mlp at batch 1: leave out what the default run adds to the line: `batch64`, `attention`, "
                         "`ppcx` and `stack`")
    ap.add_argument("--no-stack", action="store_true", help="mlp at batch 1: leave out the whole-stack pass only")
    ap.add_argument("--distinct-layers", type=int, default=4,
                    help="stack: layers of each kind encoded from their own seeds; the rest are device copies of these")
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
    if args.workload == "attention":
        return run_attention(args)
    if args.workload == "stack":
        if not 1 <= args.distinct_layers <= args.layers:
            sys.exit("bench.py: --distinct-layers must be between 1 and --layers")
        return run_stack(args)

    headline = args.workload == "mlp" and args.batch == 1 and not args.only and not args.no_extras
    stack_args = prep = None
    if headline and not args.no_stack:
        # the stack's matrices are drawn, encoded and indexed in worker processes from now on (forked
        # before this process touches the GPU), beside the GPU phases of the other workloads
        stack_args = argparse.Namespace(**vars(args))
        stack_args.batch, stack_args.steps, stack_args.warmup = 64, max(3, args.steps // 10), max(2, args.warmup // 10)
        prep = StackPrep(stack_args)
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
    # matrices that are served in batches keep their packed residuals in blocks of sixteen rows,
    # the matrix-core kernel's unit; the others in blocks of the vector-ALU kernel's unit
    residual_block = args.residual_block or (16 if args.batch > GEMV_UP_TO else None)
    for i, name in enumerate(SHAPES):
        if name not in names:
            continue
        rows, cols = SHAPES[name]
        w = synth_weights(i, rows, cols)
        t0 = time.perf_counter()
        frame = codec.encode(w)
        t1 = time.perf_counter()
        tensors[name] = HipContextTensor(frame, stride=1024, device="cuda:0", fused_segment=args.segment or None,
                                         residual_block=residual_block)
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

    def measure(m, layers=layers):
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

        tensors, pair = layers[0]
        per_layer = [units_of(*layer) for layer in layers]
        units = per_layer[0]
        if pair is not None and not decode_only:
            log(f"batch {m} gate+up: one launch, tiling {pair._tiling('waves' if m <= GEMV_UP_TO else 'gemm')[0][3]}")
        ms_per_step, per_kernel_ms, launch, timing, clocks = time_launches(
            torch, per_layer, args.steps, args.warmup, args.graph,
            lambda: sorted({n_ for ts, pr in layers for n_ in names if ts[n_].error.item()}
                           | {"gate+up" for ts, pr in layers if pr is not None and pr.error.item()}))
        if args.calibrate_copy:
            calibration_copy(torch)
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
        kernel = kernel_name(decode_only, m, "+" in dom, tensors[names[0]].fused_plan["seg_len"],
                             bool(tensors[names[0]].fused.raw_interleaved))
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
                       "layer_copies": n_layers, "residual_block_rows": tensors[names[0]]._raw6_block},
            "effective_bf16_GBps": round(eff_bf16, 2),
            "tok_s_equiv": round(eff_bf16 * 1e9 / MODEL_BF16_BYTES * m, 3) if m else None,
            **clocks,
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
    if headline:
        # the other figures of the metric, timed in the same run: the MLP step at batch 64 (fused
        # GEMM on the matrix cores), the attention projections through the batch-invariant GEMM,
        # a predictive frame, and one pass through a whole resident stack
        # what the M-invariant policy (HipContextTensor(..., m_invariant=True), the MTP head's and
        # BctxLinear(batch_invariant=True)'s route: every row count through the matrix-core kernel,
        # so a row's bits do not depend on the batch) costs on the down projection at 1 and 6 rows,
        # beside the default route (1 row: the vector-ALU kernel; 6 rows: the same matrix-core kernel)
        log("M-invariant policy on down ...")
        rng6 = np.random.default_rng(11)
        x6 = torch.from_numpy(bf16_words(rng6.normal(0, 1, size=(6, SHAPES["down"][1])))).view(torch.bfloat16).cuda()
        policy = {"matrix": "down %dx%d" % SHAPES["down"], "m1_default_ms": result["per_kernel"]["down"]["ms"]}
        for key, rows_, inv in (("m1_invariant_ms", 1, True), ("m6_default_ms", 6, False), ("m6_invariant_ms", 6, True)):
            per_layer = [[("down", ["down"], lambda t=ts["down"], r=rows_, i=inv: t.linear(x6[:r], batch_invariant=i))]
                         for ts, _ in layers]
            _, per, _, _, _ = time_launches(torch, per_layer, min(args.steps, 40), min(args.warmup, 10), args.graph,
                                            lambda: sorted({"down" for ts, _ in layers if ts["down"].error.item()}))
            policy[key] = round(per["down"], 4)
        result["m_invariant_policy"] = policy
        log("batch 64 ...")
        # matrices that are served in batches keep their packed residuals in blocks of sixteen rows
        # (a load-time choice: HipContextTensor(..., residual_block=16)); here the copies are
        # re-ordered on the device
        for i, (ts, pr) in enumerate(layers):
            ts = {n_: t.clone(residual_block=16) for n_, t in ts.items()}
            layers[i] = (ts, HipLinearGroup([ts["gate"], ts["up"]]) if pr is not None else None)
        torch.cuda.empty_cache()
        b64, _ = measure(64, layers)
        result["batch64"] = b64
        b64["config"] = {"residual_block_rows": b64.pop("config")["residual_block_rows"]}
        del tensors, pair, layers
        torch.cuda.empty_cache()
        log("attention ...")
        result["attention"] = run_attention(args, as_dict=True)
        log("ppcx ...")
        result["ppcx"] = run_predictive(args, as_dict=True)
    if prep is not None:
        prep.wait()  # (before the CPU baseline takes the host's cores)
    if not args.no_cpu_baseline:
        log("timing the CPU oracle on whole frames ...")
        result["cpu_baseline"] = cpu_baseline(frames, words_of, x_words)
        result["cpu_baseline"]["host"] = host_description()
    if prep is not None:
        log("whole stack ...")
        result["stack"] = run_stack(stack_args, as_dict=True, prep=prep)
    print(json.dumps(result), flush=True)


def kernel_name(decode_only, m, grouped, seg_len, interleaved=True):
    """The kernel a launch of the workload runs (as rocprofv3 names it)."""
    # the store sink reads a 64-symbol segment's residuals at once only from an array in the frame's
    # own order; the resident array of a fused frame is in blocked order (raw_interleaved)
    ahead = "true" if seg_len == 64 and not interleaved else "false"
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


def recorded_traffic(decode_only, m, kernel, prefix=None):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE
    record (bench.py cannot read hardware counters itself), and where the figure comes from.
    The record names the kernels it measured and the digest of the device sources it was taken
    with; for another kernel or other sources the figure is withheld (None) and the reason given."""
    name = ((f"ppcx_gemv_m1_5120x17408_traffic.json" if m == 1 else f"ppcx_gemm_m{m}_5120x17408_traffic.json")
            if prefix == "ppcx" else
            "fused_store_decode_qwen27b_mlp_traffic.json" if decode_only else
            "fused_gemv_m1_qwen27b_mlp_traffic.json" if m == 1 else
            "fused_gemm_m64_qwen27b_mlp_traffic.json" if m == 64 else None)
    if name is None or not (ROOT / "profiles" / name).exists():
        return None, "no counter record for this workload"
    record = json.loads((ROOT / "profiles" / name).read_text())
    per_kernel = record.get("traffic_bytes_per_launch")
    short = "product" if prefix == "ppcx" else kernel.split("<")[0].split("::")[-1]
    if not isinstance(per_kernel, dict) or short not in per_kernel:
        return None, f"profiles/{name} holds no figure for {short}"
    if record.get("kernel_sources_sha256") != kernel_sources_sha256():
        return None, f"profiles/{name} was recorded with other kernel sources (its figure for {short}: {per_kernel[short]:.0f} B)"
    return per_kernel[short], f"recorded: profiles/{name} (rocprofv3 --pmc, same kernel sources)"


class Stamps:
    """Device timestamps between launches (grf_timestamp: a one-lane kernel that reads the device's
    constant-rate counter and its shader-clock counter in stream order).  Events cannot be recorded
    inside a captured HIP graph on this platform; these launches can, so a graph of steps with a
    stamp after every launch gives each launch's duration in the very sequence that is timed."""

    def __init__(self, torch, count):
        from georefine_amd import _native
        self.torch, self.lib = torch, _native.hip()
        self.khz = self.lib.grf_wall_clock_khz() or 100000
        self.buf = torch.zeros((count, 3), dtype=torch.int64, device="cuda")
        self.used = 0

    def mark(self):
        torch = self.torch
        if self.lib.grf_timestamp(self.buf[self.used].data_ptr(), torch.cuda.current_stream().cuda_stream):
            raise RuntimeError(self.lib.grf_last_error().decode(errors="replace"))
        self.used += 1

    def read(self):
        """(milliseconds at every mark, shader clock in MHz between the two marks farthest apart
        that ran on one compute unit -- the counters of different units do not share a zero)"""
        host = self.buf[:self.used].cpu().numpy()
        ms = host[:, 0].astype(np.float64) / self.khz
        mhz, span = 0.0, 0.0
        for unit in np.unique(host[:, 2]):
            at = np.flatnonzero(host[:, 2] == unit)
            if at.size > 1 and ms[at[-1]] - ms[at[0]] > span:
                span = ms[at[-1]] - ms[at[0]]
                mhz = float(host[at[-1], 1] - host[at[0], 1]) / (span * 1e3)
        return ms, mhz


class StampedGraph:
    """`launches` (callables, in order) captured with a stamp after each, and two stamps back to
    back first, whose distance is what a stamp itself adds to the sequence."""

    def __init__(self, torch, launches):
        self.torch = torch
        self.stamps = Stamps(torch, len(launches) + 2)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.stamps.mark()
            self.stamps.mark()
            for run in launches:
                run()
                self.stamps.mark()

    def durations(self, replays=2):
        """(ms of every launch with the stamp's share taken off, the stamp's share in ms, shader
        clock in MHz over the whole sequence, ms of the whole sequence), from the last replay."""
        for _ in range(replays):
            self.graph.replay()
        self.torch.cuda.synchronize()
        ms, mhz = self.stamps.read()
        own = ms[1] - ms[0]
        spans = np.diff(ms[1:]) - own
        whole = ms[-1] - ms[1]
        return spans, own, mhz, whole


MAX_GRAPH_LAUNCHES = 4096  # kernel nodes per captured graph


def time_launches(torch, per_layer, steps, warmup, graph, errors):
    """(ms per step, {label: ms per launch}, how the step was launched, how launches were timed,
    {shader clock, the step as the stamps see it, ...}).

    `per_layer[c]` holds the launches of a step, (label, members, callable) each, on copy c of
    the workload's matrices; step i runs on copy i mod len(per_layer), so no step finds its
    matrices in the caches.  A label may occur several times in a step (the layers of a stack):
    its figure is the mean over its launches.

    Order of events: `warmup` eager steps (they also upload tilings and let the allocator
    settle); every graph is captured -- the graphs of up to 96 consecutive steps that are timed,
    and a graph of the same steps with a device timestamp after every launch (Stamps); the timed
    graphs are replayed once more as they will be timed, untimed, so that the clocks are where
    sustained work holds them (captures leave the GPU idle for tens of milliseconds, and the first
    launches after such a gap run at a lower clock); synchronise; exactly `steps` steps are
    replayed and timed on the host clock; synchronise.  Then the stamped graph gives the
    per-launch durations: the same kernels in the same order on the same copies, so the
    launches' sum and the step agree up to what the stamps add, which is measured and taken
    off.  Without graphs (--no-graph, or a capture that fails): eager steps, and HIP events
    around single launches."""
    copies = len(per_layer)
    labels = [label for label, _, _ in per_layer[0]]
    names = list(dict.fromkeys(labels))

    def step(i):
        return [run() for _, _, run in per_layer[i % copies]]

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    bad = errors()
    if bad:
        sys.exit(f"bench.py: decoder error word set for {bad}")
    launch, wall, extra = "eager", None, {}
    per_kernel_ms = {}
    chunk = min(steps, 96, max(1, MAX_GRAPH_LAUNCHES // len(labels)))
    chunk = chunk // copies * copies or chunk  # whole turns through the copies where a step is small
    graphs, stamped = [], None
    if graph:
        # consecutive steps captured once and replayed: the launches are submitted together, which
        # takes the host's per-launch latency out of the gaps between kernels
        try:
            plan = [(chunk, steps // chunk)] + ([(steps % chunk, 1)] if steps % chunk else [])
            for length, times in plan:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    for i in range(length):
                        step(i)
                graphs.append((g, times))
            torch.cuda.synchronize()
        except Exception as exc:  # keep the eager figure
            log(f"graph capture failed ({exc}); reporting the eager steps")
            graphs = []
        if graphs:
            try:
                stamped = StampedGraph(torch, [per_layer[i % copies][j][2] for i in range(chunk)
                                               for j in range(len(labels))])
            except Exception as exc:
                log(f"stamped graph failed ({exc}); timing eager launches")
    if graphs:
        for g, times in graphs:  # untimed, as they will be timed
            for _ in range(times):
                g.replay()
        torch.cuda.synchronize()
        wall0 = time.perf_counter()
        for g, times in graphs:
            for _ in range(times):
                g.replay()
        torch.cuda.synchronize()
        wall = time.perf_counter() - wall0
        launch = "hip graph replay"
    else:
        for i in range(max(warmup, 1)):
            step(i)
        torch.cuda.synchronize()
        wall0 = time.perf_counter()
        for i in range(steps):
            step(i)
        torch.cuda.synchronize()
        wall = time.perf_counter() - wall0
    if stamped is not None:
        spans, own, mhz, whole = stamped.durations()
        spans = spans.reshape(chunk, len(labels))
        per_kernel_ms = {n_: float(np.mean([spans[:, j].mean() for j, l_ in enumerate(labels) if l_ == n_]))
                         for n_ in names}
        timing = (f"device timestamps after every launch inside a HIP graph of {chunk} consecutive steps (the "
                  f"steps that are timed, plus the stamps), over {copies} device copies of the matrices in turn; a "
                  f"stamp's own share ({own * 1e3:.1f} us) is taken off every launch")
        extra = {"sclk_mhz": round(mhz, 1), "stamp_us": round(own * 1e3, 2),
                 "step_ms_stamped_graph": round(whole / chunk, 4),
                 "launches_sum_ms": round(float(spans.sum(axis=1).mean()), 4)}
    if not per_kernel_ms:
        timing = "HIP events around single eager launches"
        n_units = len(labels)
        starts = [[torch.cuda.Event(enable_timing=True) for _ in range(n_units)] for _ in range(steps)]
        ends = [[torch.cuda.Event(enable_timing=True) for _ in range(n_units)] for _ in range(steps)]
        torch.cuda.synchronize()
        for s_ in range(steps):
            for j, (_, _, run) in enumerate(per_layer[s_ % copies]):
                starts[s_][j].record()
                run()
                ends[s_][j].record()
        torch.cuda.synchronize()
        per_kernel_ms = {n_: float(np.mean([starts[s_][j].elapsed_time(ends[s_][j]) for s_ in range(steps)
                                            for j, l_ in enumerate(labels) if l_ == n_])) for n_ in names}
    bad = errors()
    if bad:
        sys.exit(f"bench.py: decoder error word set for {bad}")
    return wall / steps * 1e3, per_kernel_ms, launch, timing, extra


if __name__ == "__main__":
    main()

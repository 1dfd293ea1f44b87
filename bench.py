#!/usr/bin/env python3
"""Benchmark of the int8 quantized-inference hot path on one MI355X.

Headline workload (``--workload linear``, the default): the LLM-shaped int8
quantized Linear, M=2048, K=4096, N=11008 - int8 weights (N(0,0.02),
per-row symmetric scales) x int8 activations (N(0,1), per-token symmetric
scales), int32 accumulation, fp16 dequantized output with fp16 bias.  A "step"
is one launch of the fused GEMM+epilogue on inputs already resident in HBM.

One JSON line is printed.  Besides the driver's fields it carries
  roofline      the GEMM against the published int8 dense MFMA peak,
  cpu_baseline  Lucid's CPU pass structure (dequantize weight -> float GEMM ->
                bias), restated in oracle/, timed on the host cores on a
                bounded row sample of the same layer,
  extra         the bandwidth-bound members of the path measured in the same
                run: quantize / dequantize / min-max on the 4096x4096x16
                round-trip tensor against the 8 TB/s HBM peak, and the
                decode-shaped Linears (M = 1, 16) against HBM, and the int8
                ResNet-50 (batch 32) in images/s.

Timing: HIP events recorded on the stream the kernels are launched on (the
default stream), through the library's own C ABI.  No PyTorch anywhere.
"""

from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X published dense int8 MFMA peak, TOP/s
PEAK_HBM_GBS = 8000.0     # MI355X published HBM3E bandwidth, GB/s

# HBM bytes per launch, measured with rocprofv3 --pmc (FETCH_SIZE and WRITE_SIZE
# in separate runs, in KiB per dispatch, scaled by what the same counters read on
# the library's plain 1 GiB copy kernel: fetch x2.000, write x1.000).  The runs
# are summarised in profiles/hbm_traffic_qlinear_and_quantize.md.
MEASURED_TRAFFIC_BYTES = {
    "quantize_per_channel_i8": int((2.0 * 524577 + 262144) * 1024),
    "dequantize_per_channel_i8": int((2.0 * 131350 + 1048712) * 1024),
    "minmax_per_channel": int((2.0 * 524317 + 257) * 1024),
}


# The headline Linear's HBM traffic depends on the tile shape, so each figure is kept with the
# tile_config (lq_last_tile_config) it was measured under and is reported only when the run
# resolves to that same configuration (null otherwise: a stale figure would mislead).
LINEAR_TRAFFIC_BY_TILE_CONFIG = {
    0x10d: int((2.0 * 57280.4 + 54085.0) * 1024),                       # one launch of 256x352 tiles, eight wavefronts
    0x104: int((2.0 * 96504 + 44032) * 1024),                           # one launch of 128x256 tiles
    0x20010b: int((2.0 * (49357.0 + 30884.2) + 32768 + 11264) * 1024),  # 256x256 over 8192 columns + 128x256 over 2816
}


def _events(_C, n):
    evs = []
    for _ in range(n):
        e = C.c_void_p()
        _C.call("lq_event_create", C.byref(e))
        evs.append(e)
    return evs


def _elapsed_ms(_C, a, b):
    ms = C.c_float()
    _C.call("lq_event_elapsed_ms", a, b, C.byref(ms))
    return float(ms.value)


def time_launches(_C, fn, steps, warmup):
    """Returns (total ms over `steps` back-to-back launches, per-launch ms list)."""
    for _ in range(warmup):
        fn()
    _C.call("lq_sync", None)
    evs = _events(_C, steps + 1)
    _C.call("lq_event_record", evs[0], None)
    for i in range(steps):
        fn()
        _C.call("lq_event_record", evs[i + 1], None)
    _C.call("lq_event_sync", evs[steps])
    per = [_elapsed_ms(_C, evs[i], evs[i + 1]) for i in range(steps)]
    total = _elapsed_ms(_C, evs[0], evs[steps])
    for e in evs:
        _C.call("lq_event_destroy", e)
    return total, per


def time_in_graph(L, _C, fn, steps, per_graph=20):
    """Average milliseconds per call of `fn` when `per_graph` calls are captured into a HIP
    graph and the graph is replayed `steps` times between one pair of events: the rate of
    short kernels without the interpreter's gap between launches."""
    fn()
    if EAGER_ONLY:  # no graph launch under a tracer: the same calls, driven from Python
        def many():
            for _ in range(per_graph):
                fn()
        total, _ = time_launches(_C, many, steps, 2)
        return total / (steps * per_graph)
    with L.graph.capture() as g:
        for _ in range(per_graph):
            fn()
    for _ in range(5):
        g.replay()
    total, _ = time_launches(_C, g.replay, steps, 2)
    g.destroy()
    return total / (steps * per_graph)


def make_linear(L, Q, _C, _ops, M, K, N, seed):
    """Synthetic layer of the benchmark's shape, quantized on the device with
    the library's own kernels."""
    wf = L.Tensor.empty((N, K), L.float32, "hip")
    _C.call("lq_fill_normal", wf.data_ptr, N * K, seed, 0.0, 1.0, None)
    # N(0, 0.02): scale the unit normals through a dequantize-free route - the
    # per-row symmetric scale absorbs the factor, so quantize the unit normals
    # and multiply the scales instead.
    mn, mx = Q.minmax(wf, ch_axis=0)
    ws, wz = Q.calculate_qparams(mn, mx, Q.per_channel_symmetric, Q.qint8)
    wq = Q.quantize(wf, ws, wz, Q.qint8, ch_axis=0)
    ws = L.tensor(ws.numpy() * np.float32(0.02), device="hip")
    x = L.Tensor.empty((M, K), L.float32, "hip")
    _C.call("lq_fill_normal", x.data_ptr, M * K, seed + 1, 0.0, 1.0, None)
    xmn, xmx = Q.minmax(x, ch_axis=0)
    xs, xz = Q.calculate_qparams(xmn, xmx, Q.per_channel_symmetric, Q.qint8)
    xq = Q.quantize(x, xs, xz, Q.qint8, ch_axis=0)
    rng = np.random.default_rng(seed)
    bias = L.tensor((rng.standard_normal(N) * 0.02).astype(np.float16), device="hip")
    out = L.Tensor.empty((M, N), L.float16, "hip")
    return dict(x=x, xq=xq, xs=xs, wq=wq, ws=ws, bias=bias, out=out)


def sample_for_verification(t, M, N, seed, rows=32):
    """Host copies of `rows` sampled rows of the timed output and of everything that determines
    them (their activation codes and scales, the whole weight matrix, scales, bias)."""
    rng = np.random.default_rng(seed + 100)
    idx = np.unique(np.concatenate([rng.integers(0, M, rows), [0, M - 1]]))
    out = t["out"].numpy()
    return dict(rows=idx, out=out[idx].copy(), xq=t["xq"].numpy()[idx].copy(), xs=t["xs"].numpy()[idx].copy(),
                wq=t["wq"].numpy(), ws=t["ws"].numpy(), bias=t["bias"].numpy())


def verify_linear_sample(v):
    """The sampled rows of the timed float16 output against the oracle's integer formulation
    (bit for bit).  Called from the cpu_baseline leg only."""
    import oracle as O

    exp = O.qlinear(v["xq"], v["wq"], 0, v["xs"], v["ws"], bias=v["bias"], out_mode=O.OUT_F16)
    same = np.array_equal(v["out"].view(np.uint16), exp.view(np.uint16))
    return {"rows_checked": int(len(v["rows"])), "columns": int(exp.shape[1]), "bit_exact": bool(same)}


def bench_linear(L, Q, _C, _ops, M, K, N, steps, warmup, seed=1, keep_verify_sample=False):
    t = make_linear(L, Q, _C, _ops, M, K, N, seed)

    def step(repeat=1):
        _ops.qlinear_i8(t["xq"], t["wq"], a_scale=t["xs"], w_scale=t["ws"], bias=t["bias"],
                        out_mode=_ops.OUT_F16, out=t["out"], repeat=repeat)

    # Let the clock settle first: after idling (the uploads and quantization above are light
    # work) the part takes tens of milliseconds of load to reach the state it then holds, and
    # a dozen 80 us warm-up launches end before that.  Untimed, like the warm-up steps.
    step()
    settle = 500
    step(settle)
    _C.call("lq_sync", None)
    # per-launch event pairs give the spread; the average launch duration comes
    # from `steps` launches issued back to back from native code between one
    # pair of events, so that no host-side gap is charged to the kernel
    _, per = time_launches(_C, step, steps, warmup)
    total, _ = time_launches(_C, lambda: step(steps), 1, 1)
    ops = 2.0 * M * K * N
    bytes_alg = N * K + M * K + 2 * M * N + 4 * N + 4 * M + 2 * N
    avg_ms = total / steps
    # what the autotuner settled on (shape | schedule << 8 | leading 256-column tiles << 16)
    tile_config = int(_C.call("lq_last_tile_config"))
    split = None
    if tile_config >> 16:
        # two kernels per step: the first NA columns on 256x256 tiles, the rest on another
        # shape.  Time the first (dominant) one alone: the same kernel on the same operands.
        NA = (tile_config >> 16) * 256
        sub = L.Tensor.empty((M, NA), L.float16, "hip")

        def first(repeat=1):
            # the leading NA rows of the weight are a contiguous prefix, so the prefix of the
            # scale / bias arrays and a narrower output describe exactly region A
            _ops.qlinear_i8(t["xq"], t["wq_head"], a_scale=t["xs"], w_scale=t["ws_head"], bias=t["bias_head"],
                            out_mode=_ops.OUT_F16, out=sub, repeat=repeat, path=1,
                            tile_config=(tile_config & 0xff) | 0x100)

        t["wq_head"] = t["wq"].narrow_rows(NA)
        t["ws_head"], t["bias_head"] = t["ws"].narrow_rows(NA), t["bias"].narrow_rows(NA)
        first()
        tot_a, _ = time_launches(_C, lambda: first(steps), 1, 1)
        split = dict(columns=NA, ops=2.0 * M * K * NA, avg_ms=tot_a / steps)
    verify = None
    if keep_verify_sample:
        # what the timed launches left in `out`, with the operands of the same rows: checked
        # against the CPU restatement in the cpu_baseline leg (sample_for_verification)
        verify = sample_for_verification(t, M, N, seed)
    return dict(tile_config=tile_config, split=split, verify=verify, total_ms=total, avg_kernel_ms=avg_ms, median_ms=float(np.median(per)),
                p95_ms=float(np.percentile(per, 95)), ops=ops, bytes=bytes_alg,
                tops=ops / (total / steps) / 1e9, kernel_tops=ops / avg_ms / 1e9,
                gbs=bytes_alg / avg_ms / 1e6, tensors=t)


def zero_operand_rate(L, _C, _ops, t, M, K, N):
    """TOP/s of the headline launch with every activation and weight code zero (scales, bias and
    output form unchanged): how fast the kernel's structure runs when the matrix cores draw the
    least power.  A diagnostic beside the timed figure."""
    xz = L.Tensor.empty((M, K), L.int8, "hip")
    wz = L.Tensor.empty((N, K), L.int8, "hip")
    _C.call("lq_fill_bytes", xz.data_ptr, 0, M * K, None)
    _C.call("lq_fill_bytes", wz.data_ptr, 0, N * K, None)
    scratch = L.Tensor.empty((M, N), L.float16, "hip")

    def step(repeat=1):
        _ops.qlinear_i8(xz, wz, a_scale=t["xs"], w_scale=t["ws"], bias=t["bias"], out_mode=_ops.OUT_F16,
                        out=scratch, repeat=repeat)

    step()
    step(300)
    _C.call("lq_sync", None)
    total, _ = time_launches(_C, lambda: step(200), 1, 1)
    return 2.0 * M * K * N / (total / 200) / 1e9


def bench_linear_cold_weights(L, _C, _ops, t, M, K, N, steps):
    """The decode-shaped layer with weights that are NOT resident in the 256 MB last-level
    cache: the launches cycle through enough copies of the weight matrix to exceed it, as the
    layers of a real model do, replayed from a HIP graph so that no host gap is charged.
    Returns the average microseconds per launch."""
    copies = int(320e6 // (N * K)) + 2
    ws = [t["wq"]] + [t["wq"].clone() for _ in range(copies - 1)]

    def cycle():
        for w in ws:
            _ops.qlinear_i8(t["xq"], w, a_scale=t["xs"], w_scale=t["ws"], bias=t["bias"],
                            out_mode=_ops.OUT_F16, out=t["out"])

    g = _Replay(L, cycle)  # a graph replay, or the same launches from Python under --eager
    for _ in range(20):
        g.run()
    total, _ = time_launches(_C, g.run, steps, 3)
    g.destroy()
    return total / (steps * copies) * 1e3


def probe_mfma_ceiling(L, _C, xq, wq, ms_target=40.0, entry="lq_probe_mfma_i8"):
    """TOP/s of a loop of nothing but int8 MFMAs over register operands taken from
    the benchmark's own activation and weight codes (two wavefronts per SIMD, eight
    independent accumulators each): what the matrix cores sustain for this data under
    the board's power limit, before any data movement.  Long enough (tens of ms) for
    the clock to settle."""
    sink = L.Tensor.empty((1,), L.int32, "hip")
    ops = C.c_double()
    nbytes = min(xq.numel, wq.numel)

    def run(iters):
        evs = _events(_C, 2)
        _C.call("lq_event_record", evs[0], None)
        _C.call(entry, xq.data_ptr, wq.data_ptr, nbytes, iters, sink.data_ptr, C.byref(ops), None)
        _C.call("lq_event_record", evs[1], None)
        _C.call("lq_event_sync", evs[1])
        ms = _elapsed_ms(_C, evs[0], evs[1])
        for e in evs:
            _C.call("lq_event_destroy", e)
        return ms

    ms = run(2000)
    iters = int(max(2000, min(2_000_000, 2000 * ms_target / max(ms, 1e-3))))
    run(iters)
    ms = run(iters)
    return ops.value / ms / 1e9


def bench_act_quant_plus_linear(L, Q, _C, _ops, t, M, K, N, steps, warmup):
    """The same layer with the dynamic per-token activation quantization in the timed
    region.  Two launches: one pass over x that takes each row's min / max, qparams and
    codes, then the GEMM; and, beside it, the four launches of the separate operators
    (min/max -> qparams -> quantize -> GEMM), same bits."""
    mn = L.Tensor.empty((M,), L.float32, "hip")
    mx = L.Tensor.empty((M,), L.float32, "hip")
    s = L.Tensor.empty((M,), L.float32, "hip")
    z = L.Tensor.empty((M,), L.float32, "hip")
    xq = L.Tensor.empty((M, K), L.int8, "hip")

    def gemm():
        _ops.qlinear_i8(xq, t["wq"], a_scale=s, w_scale=t["ws"], bias=t["bias"],
                        out_mode=_ops.OUT_F16, out=t["out"])

    def fused():
        _C.call("lq_quantize_rows_dynamic_i8", t["x"].data_ptr, M, K, 1, -128, 127, 1, 1e-8, 0, s.data_ptr,
                z.data_ptr, None, None, xq.data_ptr, None)
        gemm()

    def separate():
        _C.call("lq_minmax", t["x"].data_ptr, 1, M, K, mn.data_ptr, mx.data_ptr, None)
        _C.call("lq_calc_qparams", mn.data_ptr, mx.data_ptr, M, 1, -128, 127, 1, 1e-8, s.data_ptr,
                z.data_ptr, None)
        _C.call("lq_quantize", t["x"].data_ptr, xq.data_ptr, _C.I8, 0, 1, M, K, s.data_ptr,
                z.data_ptr, 0, -128, 127, None)
        gemm()

    total, _ = time_launches(_C, fused, steps, warmup)
    total4, _ = time_launches(_C, separate, steps, warmup)
    ops = 2.0 * M * K * N
    return ops / (total / steps) / 1e9, ops / (total4 / steps) / 1e9


def bench_linear_from_host(L, Q, _C, _ops, t, M, K, N, steps):
    """The same layer when the caller holds host buffers: float32 activations
    uploaded (pageable memory, as numpy hands them over), dynamic activation
    quantization, GEMM, fp16 result downloaded.  Wall clock per call."""
    rng = np.random.default_rng(7)
    xh = rng.standard_normal((M, K)).astype(np.float32)
    outh = np.empty((M, N), np.float16)
    mn = L.Tensor.empty((M,), L.float32, "hip")
    mx = L.Tensor.empty((M,), L.float32, "hip")
    s = L.Tensor.empty((M,), L.float32, "hip")
    z = L.Tensor.empty((M,), L.float32, "hip")
    xq = L.Tensor.empty((M, K), L.int8, "hip")
    times = []
    for _ in range(steps + 2):
        t0 = time.perf_counter()
        _C.call("lq_h2d", t["x"].data_ptr, xh.ctypes.data, xh.nbytes, None)
        _C.call("lq_minmax", t["x"].data_ptr, 1, M, K, mn.data_ptr, mx.data_ptr, None)
        _C.call("lq_calc_qparams", mn.data_ptr, mx.data_ptr, M, 1, -128, 127, 1, 1e-8, s.data_ptr,
                z.data_ptr, None)
        _C.call("lq_quantize", t["x"].data_ptr, xq.data_ptr, _C.I8, 0, 1, M, K, s.data_ptr,
                z.data_ptr, 0, -128, 127, None)
        _ops.qlinear_i8(xq, t["wq"], a_scale=s, w_scale=t["ws"], bias=t["bias"],
                        out_mode=_ops.OUT_F16, out=t["out"])
        _C.call("lq_d2h", outh.ctypes.data, t["out"].data_ptr, outh.nbytes, None)
        times.append(time.perf_counter() - t0)
    dt = float(np.median(times[2:]))
    return {"ms_per_call": round(dt * 1e3, 3), "TOP/s": round(2.0 * M * K * N / dt / 1e12, 2),
            "host_bytes_moved": int(xh.nbytes + outh.nbytes),
            "host_GB/s": round((xh.nbytes + outh.nbytes) / dt / 1e9, 2)}


def bench_quant_roundtrip(L, Q, _C, steps, warmup):
    """Config: 4096 x 4096 x 16 float32, N(0,1) with 0.1 % outliers x20;
    per-channel symmetric int8 along dim 0, then per-tensor affine."""
    shape = (4096, 4096, 16)
    n = int(np.prod(shape))
    Cn, inner = shape[0], shape[1] * shape[2]
    x = L.Tensor.empty(shape, L.float32, "hip")
    _C.call("lq_fill_normal", x.data_ptr, n, 2, 0.001, 20.0, None)
    mn, mx = Q.minmax(x, ch_axis=0)
    s, z = Q.calculate_qparams(mn, mx, Q.per_channel_symmetric, Q.qint8)
    q = L.Tensor.empty(shape, L.int8, "hip")
    dq = L.Tensor.empty(shape, L.float32, "hip")
    gmn, gmx = Q.minmax(x)
    ts, tz = Q.calculate_qparams(gmn, gmx, Q.per_tensor_affine, Q.quint8)
    q16 = L.Tensor.empty(shape, L.int16, "hip")

    cases = {
        "minmax_per_channel": (4 * n, lambda: _C.call(
            "lq_minmax", x.data_ptr, 1, Cn, inner, mn.data_ptr, mx.data_ptr, None)),
        "minmax_per_tensor": (4 * n, lambda: _C.call(
            "lq_minmax", x.data_ptr, 1, 1, n, gmn.data_ptr, gmx.data_ptr, None)),
        "quantize_per_channel_i8": (5 * n, lambda: _C.call(
            "lq_quantize", x.data_ptr, q.data_ptr, _C.I8, 0, 1, Cn, inner, s.data_ptr, z.data_ptr,
            0, -128, 127, None)),
        "dequantize_per_channel_i8": (5 * n, lambda: _C.call(
            "lq_dequantize", q.data_ptr, _C.I8, 0, dq.data_ptr, 1, Cn, inner, s.data_ptr,
            z.data_ptr, 0, None)),
        "quantize_per_tensor_quint8_i16": (6 * n, lambda: _C.call(
            "lq_quantize", x.data_ptr, q16.data_ptr, _C.I16, 0, 1, 1, n, ts.data_ptr, tz.data_ptr,
            0, 0, 255, None)),
        "dequantize_per_tensor_quint8_i16": (6 * n, lambda: _C.call(
            "lq_dequantize", q16.data_ptr, _C.I16, 0, dq.data_ptr, 1, 1, n, ts.data_ptr,
            tz.data_ptr, 0, None)),
        "copy_kernel": (8 * n, lambda: _C.call(
            "lq_copy_kernel", dq.data_ptr, x.data_ptr, 4 * n, None)),
    }
    out = {}
    for name, (nbytes, fn) in cases.items():
        _, per = time_launches(_C, fn, steps, warmup)
        med = float(np.median(per))
        out[name] = {"us": round(med * 1e3, 1), "GB/s": round(nbytes / med / 1e6, 1),
                     "frac_of_8TBs": round(nbytes / med / 1e6 / PEAK_HBM_GBS, 4),
                     "bytes": nbytes, "traffic": MEASURED_TRAFFIC_BYTES.get(name)}
    # a slice of what the timed kernels left behind (channel 1234: input, codes, the per-channel
    # dequantization of those codes), checked against the CPU restatement in the cpu_baseline leg
    ch = 1234
    _C.call("lq_dequantize", q.data_ptr, _C.I8, 0, dq.data_ptr, 1, Cn, inner, s.data_ptr, z.data_ptr, 0, None)
    _C.call("lq_sync", None)
    QUANT_VERIFY.update(x=x.row_range(ch, ch + 1).numpy().reshape(-1), q=q.row_range(ch, ch + 1).numpy().reshape(-1),
                        dq=dq.row_range(ch, ch + 1).numpy().reshape(-1), s=s.numpy()[ch:ch + 1], z=z.numpy()[ch:ch + 1])
    return out


QUANT_VERIFY = {}


def verify_quant_slice():
    """One channel of the timed quantize / dequantize outputs against the oracle, bit for bit."""
    import oracle as O

    v = QUANT_VERIFY
    if not v:
        return None
    codes = O.quantize(v["x"], v["s"], v["z"], -128, 127)
    back = O.dequantize(codes, v["s"], v["z"])
    return {"elements_checked": int(v["x"].size),
            "bit_exact": bool(np.array_equal(codes.astype(np.int8), v["q"]) and
                              np.array_equal(back.view(np.uint32), v["dq"].view(np.uint32)))}


def _acc_digest(c):
    """Two position-weighted int64 sums of an int32 matrix: equal digests = equal accumulators
    (up to collisions no kernel bug would hit)."""
    c = np.asarray(c).astype(np.int64)
    wr = (np.arange(c.shape[0], dtype=np.int64) * 31 % 1009 + 1)[:, None]
    wc = (np.arange(c.shape[1], dtype=np.int64) * 17 % 1013 + 1)[None, :]
    return [int(c.sum()), int((c * wr * wc).sum())]


def vendor_child(path, steps, warmup):
    """Child process of --vendor-yardstick: torch only (its own copy of the HIP runtime cannot
    share a process with this library's), operands from the .npz the parent wrote."""
    import torch

    z = np.load(path)
    a, w = torch.from_numpy(z["a"]).cuda(), torch.from_numpy(z["w"]).cuda()
    c = torch._int_mm(a, w.t())
    digest = _acc_digest(c.cpu().numpy())
    for _ in range(warmup):
        torch._int_mm(a, w.t())
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(steps):
        torch._int_mm(a, w.t())
    e1.record()
    torch.cuda.synchronize()
    print(json.dumps({"ms": e0.elapsed_time(e1) / steps, "digest": digest}))
    return 0


def vendor_yardstick(L, Q, _C, _ops, steps, warmup):
    """The vendor library's int8 x int8 -> int32 GEMM (hipBLASLt behind ``torch._int_mm``) on the
    very codes this library's kernel is timed on: the matrix cores' clock depends on the operand
    data, so only the same codes compare.  The vendor call writes raw int32 accumulators; this
    library is timed both with its fused fp16 epilogue and writing the accumulators.  torch runs
    in a child process; this process idles meanwhile."""
    import subprocess
    import tempfile

    out = {}
    for (M, K, N) in ((2048, 4096, 11008), (2048, 4096, 8192), (8192, 4096, 11008), (8192, 8192, 8192)):
        r = bench_linear(L, Q, _C, _ops, M, K, N, steps, warmup)
        t = r["tensors"]
        acc = L.Tensor.empty((M, N), L.int32, "hip")
        _ops.qlinear_i8(t["xq"], t["wq"], out_mode=_ops.OUT_ACC_I32, out=acc)
        tot, _ = time_launches(_C, lambda: _ops.qlinear_i8(t["xq"], t["wq"], out_mode=_ops.OUT_ACC_I32, out=acc,
                                                           repeat=steps), 1, 1)
        digest = _acc_digest(acc.numpy())
        with tempfile.TemporaryDirectory() as d:
            path = os.path.join(d, "operands.npz")
            np.savez(path, a=t["xq"].numpy(), w=t["wq"].numpy())
            child = subprocess.run([sys.executable, os.path.abspath(__file__), "--vendor-child", path,
                                    "--steps", str(steps), "--warmup", str(warmup)],
                                   capture_output=True, text=True, timeout=600)
        if child.returncode != 0:
            raise RuntimeError("vendor yardstick child failed: " + child.stderr[-2000:])
        v = json.loads(child.stdout.strip().splitlines()[-1])
        out[f"M{M}_K{K}_N{N}"] = {
            "this_library_fp16_epilogue_TOP/s": round(r["kernel_tops"], 1),
            "this_library_int32_accumulators_TOP/s": round(r["ops"] / (tot / steps) / 1e9, 1),
            "vendor_int32_accumulators_TOP/s": round(r["ops"] / v["ms"] / 1e9, 1),
            "vendor_us": round(v["ms"] * 1e3, 1), "accumulators_equal": v["digest"] == digest}
        del r, t, acc
    return out


EAGER_ONLY = False  # --eager: time Python-driven launches where a graph replay is timed by default


class _Replay:
    """`fn` captured into a HIP graph (default), or `fn` itself under --eager."""

    def __init__(self, L, fn):
        self.graph = None
        if EAGER_ONLY:
            self.run, self.how = fn, "eager launches"
        else:
            with L.graph.capture() as g:
                fn()
            self.graph, self.run, self.how = g, g.replay, "hip graph replay"

    def destroy(self):
        if self.graph is not None:
            self.graph.destroy()


def bench_resnet50(L, _C, steps, warmup):
    """int8 static-quantized ResNet-50, batch 32, 3x224x224 uniform[0,1] inputs,
    random He-normal weights with BatchNorm folded, fixed calibration grids.  The
    forward (53 convolutions, 16 residual joins, pooling, classifier: ~75
    launches) is captured once into a HIP graph and replayed."""
    import workloads as W

    model = W.QResNet50()
    rng = np.random.default_rng(0)
    batch = 32
    x = L.tensor(rng.uniform(0, 1, (batch, 3, 224, 224)).astype(np.float32), device="hip")
    y = model(x)  # eager warm-up caches host-side scalars
    g = _Replay(L, lambda: model(x))
    total, per = time_launches(_C, g.run, steps, warmup)
    ms = total / steps
    gmacs = W.resnet50_conv_gmacs(batch)
    out = {"images_per_s": round(batch / ms * 1e3, 1), "ms_per_batch": round(ms, 4), "batch": batch,
           "int8_TOP/s": round(2 * gmacs / ms, 2), "GMAC_per_batch": round(gmacs, 2),
           "p95_ms": round(float(np.percentile(per, 95)), 4), "launch": g.how}
    ref = y.numpy()
    assert np.isfinite(ref).all()
    g.destroy()
    if not EAGER_ONLY:
        # the same batch as two halves, captured as two parallel branches of one graph: a forward is
        # ~60 short dependent launches, and one half's ramp-up and drain gaps are filled by the
        # other's kernels.  Same result, bit for bit
        # (static quantization: an image's result does not depend on its neighbours).
        model(x.row_range(0, batch // 2))
        sg = L.graph.capture_split(model, x, 2)
        total2, per2 = time_launches(_C, sg.replay, steps, warmup)
        ms2 = total2 / steps
        L.synchronize()
        assert np.array_equal(sg.output.numpy(), ref)
        sg.destroy()
        out["one_graph"] = {"images_per_s": out["images_per_s"], "ms_per_batch": out["ms_per_batch"],
                            "p95_ms": out["p95_ms"]}
        if ms2 < ms:
            out.update({"images_per_s": round(batch / ms2 * 1e3, 1), "ms_per_batch": round(ms2, 4),
                        "int8_TOP/s": round(2 * gmacs / ms2, 2), "p95_ms": round(float(np.percentile(per2, 95)), 4),
                        "launch": "hip graph replay, batch halves as two parallel branches"})
    return out


def bench_vit_b16(L, _C, steps, warmup):
    """Dynamic-quantized ViT-B/16, batch 64, 3x224x224 uniform[0,1] inputs, random
    N(0, 0.02) weights: all Linears W8A8 with runtime activation qparams; patch
    embedding, LayerNorm, attention, GELU and residuals float32.  Captured once
    into a HIP graph and replayed; eager time beside it."""
    import workloads as W

    model = W.QViT()
    rng = np.random.default_rng(0)
    batch = 64
    x = L.tensor(rng.uniform(0, 1, (batch, 3, 224, 224)).astype(np.float32), device="hip")
    y = model(x)
    eager_total, _ = time_launches(_C, lambda: model(x), max(3, steps // 4), 1)
    eager_ms = eager_total / max(3, steps // 4)
    g = _Replay(L, lambda: model(x))
    total, per = time_launches(_C, g.run, steps, warmup)
    ms = total / steps
    gops = W.vit_linear_gops(batch=batch)
    out = {"images_per_s": round(batch / ms * 1e3, 1), "ms_per_batch": round(ms, 4), "batch": batch,
           "eager_ms_per_batch": round(eager_ms, 4),
           "linear_int8_TOP/s_end_to_end": round(gops / ms, 2), "linear_GOP_per_batch": round(gops, 1),
           "p95_ms": round(float(np.percentile(per, 95)), 4), "launch": g.how}
    assert np.isfinite(y.numpy()).all()
    g.destroy()
    return out


def bench_dynamic_mlp(L, Q, _C, steps, warmup):
    """Dynamic-quantized MLP Linear(784,256)-ReLU-Linear(256,10), batch 64
    (launch-latency bound: 0.43 MOP).  One forward is ONE launch (layer 1 as 64 blocks, each taking
    the input's min / max, qparams and its rows' codes itself; the last block to finish reduces
    the hidden activation's range and runs layer 2) when driven from Python, which is bound by
    what a launch costs the host; a captured graph holds the two layers as two launches (shorter
    kernels, and a replay pays the launch cost once either way).  Eager = Python-driven forwards
    back to back; graph = the forward replayed from a HIP graph."""
    import lucid_amd.nn as nn

    rng = np.random.default_rng(1)
    layers = []
    for fin, fout in ((784, 256), (256, 10)):
        lin = nn.Linear(fin, fout)
        lin.register_buffer("weight", L.tensor((rng.standard_normal((fout, fin)) * 0.05).astype(np.float32)))
        lin.register_buffer("bias", L.tensor((rng.standard_normal(fout) * 0.05).astype(np.float32)))
        layers.append(lin)
    model = Q.quantize_dynamic(nn.Sequential(layers[0], nn.ReLU(), layers[1]))
    x = L.tensor(rng.standard_normal((64, 784)).astype(np.float32), device="hip")
    y = model(x)
    total, _ = time_launches(_C, lambda: model(x), steps, warmup)
    eager_us = total / steps * 1e3
    g = _Replay(L, lambda: model(x))
    total, _ = time_launches(_C, g.run, steps, warmup)
    graph_us = total / steps * 1e3
    assert np.isfinite(y.numpy()).all()
    g.destroy()
    return {"eager_us_per_forward": round(eager_us, 1), "graph_us_per_forward": round(graph_us, 1),
            "launches_per_forward": {"eager": 1, "graph": 2}}


def bench_weight_only(L, _C, steps, warmup, K=4096, N=11008, gs=64):
    """Group-wise weight-only Linear (float32 activations, int4 / int8 weights decoded
    inside the product) at decode-sized M: the launch streams the packed weight once, so
    the figure of merit is bytes of (codes + scales + biases) per second."""
    from lucid_amd.quantization import _qgemm

    rng = np.random.default_rng(9)
    w = L.tensor((rng.standard_normal((N, K)) * 0.05).astype(np.float32), device="hip")
    out = {}
    for bits in (4, 8):
        packed, scales, biases = _qgemm.quantize(w, gs, bits)
        nbytes = N * K * bits // 8 + 2 * 4 * N * (K // gs)
        for m in (1, 16):
            x = L.tensor(rng.standard_normal((m, K)).astype(np.float32), device="hip")
            res = L.Tensor.empty((m, N), L.float32, "hip")
            fn = lambda: _C.call("lq_wq_matmul", x.data_ptr, packed.data_ptr, scales.data_ptr, biases.data_ptr,
                                 m, N, K, gs, bits, res.data_ptr, None)
            # us: launches replayed back to back from a HIP graph (the kernel's own rate);
            # bracketed_launch_median_us: each launch driven from Python between its own events
            us = time_in_graph(L, _C, fn, max(10, steps // 2)) * 1e3
            _, per = time_launches(_C, fn, steps, warmup)
            gbs = nbytes / (us * 1e-6) / 1e9
            # cold: the launches of one graph cycle through copies of the packed weight that together
            # exceed the 256 MB last-level cache, so every byte comes from HBM (what a model's layers see)
            copies = int(320e6 // nbytes) + 2
            sets = [(packed, scales, biases)] + [(packed.clone(), scales.clone(), biases.clone()) for _ in range(copies - 1)]
            def cycle():
                for (pk, sc, bi) in sets:
                    _C.call("lq_wq_matmul", x.data_ptr, pk.data_ptr, sc.data_ptr, bi.data_ptr, m, N, K, gs, bits,
                            res.data_ptr, None)

            g = _Replay(L, cycle)
            for _ in range(5):
                g.run()
            tot, _ = time_launches(_C, g.run, max(10, steps // 2), 2)
            g.destroy()
            cold_us = tot / (max(10, steps // 2) * copies) * 1e3
            del sets
            out[f"w{bits}_m{m}"] = {"us_weights_in_llc": round(us, 2),
                                    "bracketed_launch_median_us": round(float(np.median(per)) * 1e3, 2),
                                    "GB/s_weights_in_llc": round(gbs, 1),
                                    "frac_of_8TBs_llc_resident": round(gbs / PEAK_HBM_GBS, 4),
                                    "us": round(cold_us, 2), "GB/s": round(nbytes / cold_us / 1e3, 1),
                                    "frac_of_8TBs": round(nbytes / cold_us / 1e3 / PEAK_HBM_GBS, 4), "bytes": nbytes}
    return out


def bench_breadth(L, Q, _C, steps, warmup):
    """HBM-bound members of the module breadth against 8 TB/s: the int8 embedding lookup
    (1 B read + 4 B written per element gathered, plus 8 B per row of scale / zero point)
    and a quantized activation on codes (1 B read + 1 B written per element)."""
    import lucid_amd.nn as nn
    import lucid_amd.nn.quantized as nnq

    rng = np.random.default_rng(11)
    out = {}
    num, dim, n_idx = 50_000, 768, 64 * 512
    emb = nnq.Embedding.from_float(nn.Embedding(num, dim))
    idx = L.tensor(rng.integers(0, num, (64, 512)).astype(np.int64), device="hip")
    res = L.Tensor.empty((64, 512, dim), L.float32, "hip")

    def lookup():
        _C.call("lq_embedding_i8", emb.weight_int8.data_ptr, emb.weight_scale.data_ptr,
                emb.weight_zero_point.data_ptr, num, dim, idx.data_ptr, 1, n_idx, -1, res.data_ptr, None)

    _, per = time_launches(_C, lookup, steps, warmup)
    nbytes = n_idx * (dim * 5 + 8 + 8)
    us = float(np.median(per)) * 1e3
    out["embedding_50000x768_32768_lookups"] = {"us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1),
                                                "frac_of_8TBs": round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4),
                                                "bytes": nbytes}
    n = 1 << 28
    codes = L.Tensor.empty((n,), L.int8, "hip")
    _C.call("lq_fill_uniform_i8", codes.data_ptr, n, 5, -128, 127, None)
    dst = L.Tensor.empty((n,), L.int8, "hip")
    s_in, z_in = L.tensor(np.float32(0.05), device="hip"), L.tensor(np.float32(128.0), device="hip")
    s_out, z_out = L.tensor(np.float32(1 / 255), device="hip"), L.tensor(np.float32(0.0), device="hip")

    def act():
        _C.call("lq_act_requant_i8", 0, 0.0, codes.data_ptr, -128, s_in.data_ptr, z_in.data_ptr, n,
                s_out.data_ptr, z_out.data_ptr, 0, 255, -128, dst.data_ptr, None)

    _, per = time_launches(_C, act, max(5, steps // 5), 2)
    us = float(np.median(per)) * 1e3
    out["sigmoid_on_codes_256Mi"] = {"us": round(us, 2), "GB/s": round(2 * n / us / 1e3, 1),
                                     "frac_of_8TBs": round(2 * n / us / 1e3 / PEAK_HBM_GBS, 4), "bytes": 2 * n}
    del codes, dst
    # a video-sized volumetric layer: 4 x 64 x 16 x 56 x 56 -> 64 channels, 3 x 3 x 3: one launch
    # whose tile loader gathers the taps from the channels-last codes the Quantize stub leaves
    B, Cc, Co, vol = 4, 64, 64, (16, 56, 56)
    c3 = nnq.Conv3d.from_float(_calibrated(L, Q, nn.Conv3d(Cc, Co, 3, padding=1), 0.04))
    x = (rng.standard_normal((B, Cc, *vol)) * 0.8).astype(np.float32)
    xq = nnq.Quantize(L.tensor(np.float32(0.03), device="hip"), L.tensor(np.float32(128.0), device="hip"),
                      Q.quint8)(L.tensor(x, device="hip"))
    _, per = time_launches(_C, lambda: c3(xq), max(5, steps // 5), 2)
    us = float(np.median(per)) * 1e3
    M, K = B * vol[0] * vol[1] * vol[2], 27 * Cc
    out["conv3d_4x64x16x56x56_to_64_k3"] = {"us": round(us, 1), "TOP/s": round(2.0 * M * Co * K / us / 1e6, 1),
                                            "gathered_bytes_through_L2": M * K, "launches": 1}
    return out


def _calibrated(L, Q, mod, out_scale):
    """Give a float layer the observer state convert() expects: a fixed output grid."""
    mod.qconfig = Q.get_default_qconfig()
    obs = mod.qconfig.activation()
    obs(L.tensor(np.array([0.0, 255.0 * out_scale], np.float32), device="hip"))
    mod.activation_post_process = obs
    return mod


def bench_vit_linears(L, Q, _C, _ops, steps, warmup):
    """The four Linear shapes of a ViT-B/16 encoder block at batch 64 (12 608
    token rows), dynamic-quantized as nnqd.Linear does: per-tensor affine quint8
    activations from the runtime min/max, per-row symmetric int8 weights, float32
    output.  GEMM-only and whole-layer (min/max + qparams + quantize + GEMM) rates."""
    M = 64 * 197
    out = {}
    for name, K, N in (("qkv", 768, 2304), ("proj", 768, 768), ("fc1", 768, 3072), ("fc2", 3072, 768)):
        t = make_linear(L, Q, _C, _ops, M, K, N, seed=7)
        x = t["x"]
        wsum = _ops.rowsum_i8(t["wq"])
        bias = L.tensor(np.zeros(N, np.float32), device="hip")
        mn, mx = Q.minmax(x)
        xs, xz = Q.calculate_qparams(mn, mx, Q.per_tensor_affine, Q.quint8)
        xq = L.Tensor.empty((M, K), L.int8, "hip")
        y = L.Tensor.empty((M, N), L.float32, "hip")

        def quant():
            _C.call("lq_minmax", x.data_ptr, 1, 1, M * K, mn.data_ptr, mx.data_ptr, None)
            _C.call("lq_calc_qparams", mn.data_ptr, mx.data_ptr, 1, 0, 0, 255, 0, 1e-8, xs.data_ptr,
                    xz.data_ptr, None)
            _C.call("lq_quantize", x.data_ptr, xq.data_ptr, _C.I8, -128, 1, 1, M * K, xs.data_ptr,
                    xz.data_ptr, 0, 0, 255, None)

        def gemm(repeat=1):
            _ops.qlinear_i8(xq, t["wq"], a_zp=-128, a_zp_dev=xz, a_scale=xs, w_scale=t["ws"],
                            wsum=wsum, bias=bias, out_mode=_ops.OUT_F32, out=y, repeat=repeat)

        quant()
        total, _ = time_launches(_C, lambda: gemm(steps), 1, 1)
        g_ms = total / steps
        total, _ = time_launches(_C, lambda: (quant(), gemm()), steps, warmup)
        l_ms = total / steps
        ops = 2.0 * M * K * N
        out[name] = {"M": M, "K": K, "N": N, "gemm_us": round(g_ms * 1e3, 1),
                     "gemm_TOP/s": round(ops / g_ms / 1e9, 1),
                     "layer_us": round(l_ms * 1e3, 1), "layer_TOP/s": round(ops / l_ms / 1e9, 1)}
    return out


def cpu_baseline_linear(K, N, sample_rows, seed=1, reps=8):
    """Lucid's CPU pass structure for this layer (dequantize the int8 weight on
    every call, float32 GEMM, bias add), run by the oracle on `sample_rows`
    rows of the same shape."""
    import oracle as O

    rng = np.random.default_rng(seed)
    wq = rng.integers(-127, 128, (N, K)).astype(np.int8)
    ws = rng.uniform(1e-4, 3e-4, N).astype(np.float32)
    wz = np.zeros(N, np.float32)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float32)
    x = rng.standard_normal((sample_rows, K)).astype(np.float32)
    times = []
    for i in range(reps + 1):  # first call warms the library and the pages
        t0 = time.perf_counter()
        O.linear_faithful(x, wq, ws, wz, bias=bias)
        times.append(time.perf_counter() - t0)
    dt = float(np.median(times[1:]))
    # one core, on a slice of the rows (the per-call weight dequantize is the same)
    rows1 = min(sample_rows, 128)
    nthreads = O.set_threads(0)
    O.set_threads(1)
    t1 = []
    for i in range(3):
        t0 = time.perf_counter()
        O.linear_faithful(x[:rows1], wq, ws, wz, bias=bias)
        t1.append(time.perf_counter() - t0)
    O.set_threads(nthreads)
    single = {"value": round(2.0 * rows1 * K * N / float(np.median(t1)) / 1e12, 5), "unit": "TOP/s",
              "cores": 1, "sample": f"{rows1} rows, median of 3 calls"}
    return 2.0 * sample_rows * K * N / dt / 1e12, dt, sum(times) + sum(t1), nthreads, single


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="linear", choices=["linear"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="only print the MFMA-only rate for several operand distributions")
    ap.add_argument("--vendor-yardstick", action="store_true",
                    help="time the ROCm library's int8 GEMM (through torch._int_mm, if torch is importable) "
                         "on the same operand codes beside this library's; a yardstick, not a dependency")
    ap.add_argument("--only", default=None, choices=["resnet50", "vit", "decode", "mlp"],
                    help="run just this end-to-end leg and print its figures")
    ap.add_argument("--vendor-child", default=None, help=argparse.SUPPRESS)
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="also run the plain 1 GiB copy kernel a few times: the known-size dispatch that "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings of the other kernels are scaled by")
    ap.add_argument("--eager", action="store_true",
                    help="time Python-driven launches instead of HIP graph replays (for runs under a tracer)")
    ap.add_argument("--cpu-sample-rows", type=int, default=2048)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2

    if args.vendor_child:
        return vendor_child(args.vendor_child, args.steps, args.warmup)

    import __graft_entry__
    __graft_entry__.ensure_built()  # loads what is built; compiles only if nothing is

    import lucid_amd as L
    import lucid_amd.quantization as Q
    from lucid_amd import _C, _ops

    _C.init(0)
    global EAGER_ONLY
    EAGER_ONLY = args.eager
    M, K, N = 2048, 4096, 11008
    if args.mfma_probe:
        # the matrix cores' sustained rate by operand statistics (no data movement at all)
        res = {}
        n = 1 << 22
        a, b = L.Tensor.empty((n,), L.int8, "hip"), L.Tensor.empty((n,), L.int8, "hip")
        for name, lo, hi in (("all_zero", 0, 0), ("uniform_-8..7", -8, 7), ("uniform_0..127", 0, 127),
                             ("uniform_-127..127", -127, 127)):
            _C.call("lq_fill_uniform_i8", a.data_ptr, n, 1, lo, hi, None)
            _C.call("lq_fill_uniform_i8", b.data_ptr, n, 2, lo, hi, None)
            res[name] = {"32x32x32": round(probe_mfma_ceiling(L, _C, a, b), 1),
                         "16x16x64": round(probe_mfma_ceiling(L, _C, a, b, entry="lq_probe_mfma_i8_k64"), 1)}
        t = make_linear(L, Q, _C, _ops, M, K, N, 1)
        res["benchmark_codes"] = {"32x32x32": round(probe_mfma_ceiling(L, _C, t["xq"], t["wq"]), 1),
                                  "16x16x64": round(probe_mfma_ceiling(L, _C, t["xq"], t["wq"],
                                                                       entry="lq_probe_mfma_i8_k64"), 1)}
        print(json.dumps({"mfma_only_tops_by_operand_data": res, "datasheet_peak_tops": PEAK_INT8_TOPS}))
        return 0
    if args.only == "decode":
        # the decode-shaped (HBM-bound) Linears alone: int8 at M = 1 / 16 and weight-only int4 / int8
        res = {}
        for m in (1, 16):
            rs = bench_linear(L, Q, _C, _ops, m, K, N, max(args.steps, 400), args.warmup, seed=3)
            cold_us = bench_linear_cold_weights(L, _C, _ops, rs["tensors"], m, K, N, max(10, args.steps // 2))
            res[f"linear_m{m}"] = {"us": round(cold_us, 2),
                                   "frac_of_8TBs": round(rs["bytes"] / cold_us / 1e3 / PEAK_HBM_GBS, 4),
                                   "us_weights_in_llc": round(rs["avg_kernel_ms"] * 1e3, 2),
                                   "frac_of_8TBs_llc_resident": round(rs["gbs"] / PEAK_HBM_GBS, 4)}
        res["weight_only_group64_k4096_n11008"] = bench_weight_only(L, _C, args.steps, args.warmup)
        print(json.dumps(res))
        return 0
    if args.only == "mlp":
        print(json.dumps({"dynamic_mlp_784_256_10_batch64": bench_dynamic_mlp(L, Q, _C, max(args.steps, 200), args.warmup)}))
        return 0
    if args.only:
        # one of the end-to-end legs alone (a clean kernel trace of one network)
        fn = {"resnet50": bench_resnet50, "vit": bench_vit_b16}[args.only]
        print(json.dumps({args.only: fn(L, _C, max(10, args.steps // 2), max(3, args.warmup // 2))}))
        return 0
    if args.vendor_yardstick:
        print(json.dumps(vendor_yardstick(L, Q, _C, _ops, args.steps, args.warmup)))
        return 0
    r = bench_linear(L, Q, _C, _ops, M, K, N, args.steps, args.warmup, keep_verify_sample=True)
    line = {
        "metric": "quantized-Linear int8 TOPS & % MFMA peak; int8 ResNet-50 images/sec",
        "value": round(r["tops"], 2),
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(r["total_ms"] / args.steps, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "int8 quantized Linear M=2048 K=4096 N=11008, per-token x per-row "
                               "scales, int32 accumulate, fp16 bias + fp16 output",
                   "device": _C.device_name()},
        "roofline": {
            "bound": "mfma",
            "achieved": round(r["kernel_tops"], 2),
            "peak": PEAK_INT8_TOPS,
            "unit": "TOP/s",
            "frac": round(r["kernel_tops"] / PEAK_INT8_TOPS, 4),
            "traffic": LINEAR_TRAFFIC_BY_TILE_CONFIG.get(r["tile_config"]),
            "kernel": {13: "qgemm_pp_kernel", 14: "qgemm_pp_kernel", 16: "qgemm_pp_kernel", 17: "qgemm_bw_kernel"}.get(
                r["tile_config"] & 0xff, "qgemm_tile_kernel"),
            "avg_kernel_us": round(r["avg_kernel_ms"] * 1e3, 2),
            "median_kernel_us": round(r["median_ms"] * 1e3, 2),
            "p95_kernel_us": round(r["p95_ms"] * 1e3, 2),
            "algorithmic_ops": r["ops"],
            "tile_config": hex(r["tile_config"]),
        },
    }
    if r["split"]:
        # a step is two launches (the tuner split the output columns between two tile shapes);
        # `achieved` above charges both, and the gap between them, to the step.  The dominant
        # kernel on its own:
        sp = r["split"]
        line["roofline"]["launches_per_step"] = 2
        line["roofline"]["dominant_kernel"] = {
            "what": f"256x256x128 tiles over the first {sp['columns']} output columns",
            "algorithmic_ops": sp["ops"], "avg_kernel_us": round(sp["avg_ms"] * 1e3, 2),
            "achieved": round(sp["ops"] / sp["avg_ms"] / 1e9, 2),
            "frac": round(sp["ops"] / sp["avg_ms"] / 1e9 / PEAK_INT8_TOPS, 4)}
    if args.traffic_calibration:
        n = 1 << 28
        src, dst = L.Tensor.empty((n,), L.float32, "hip"), L.Tensor.empty((n,), L.float32, "hip")
        _C.call("lq_fill_bytes", src.data_ptr, 1, 4 * n, None)
        for _ in range(4):
            _C.call("lq_copy_kernel", dst.data_ptr, src.data_ptr, 4 * n, None)
        _C.call("lq_sync", None)
        del src, dst
    # the same operand codes through a loop of MFMAs alone: the data-dependent ceiling
    # (v_mfma_i32_16x16x64_i8 in the kernel's own register walk: the instruction the kernel issues;
    # the 32x32x32 form, which draws more power per operation, beside it)
    ceiling = probe_mfma_ceiling(L, _C, r["tensors"]["xq"], r["tensors"]["wq"], entry="lq_probe_mfma_i8_k64")
    line["roofline"]["mfma_only_same_operands_tops"] = round(ceiling, 1)
    line["roofline"]["frac_of_mfma_only"] = round(r["kernel_tops"] / ceiling, 4)
    line["roofline"]["mfma_only_same_operands_32x32x32_tops"] = round(
        probe_mfma_ceiling(L, _C, r["tensors"]["xq"], r["tensors"]["wq"]), 1)
    # diagnostic, never the headline: the same launch on all-zero operands.  No operand bit toggles,
    # so the board's power limit does not pull the clock down and what is left is the kernel's structure.
    line["roofline"]["zero_operands_diagnostic_tops"] = round(zero_operand_rate(L, _C, _ops, r["tensors"], M, K, N), 1)
    if not args.no_extra:
        extra = {}
        fused_tops, separate_tops = bench_act_quant_plus_linear(L, Q, _C, _ops, r["tensors"], M, K, N,
                                                                args.steps, args.warmup)
        extra["linear_with_dynamic_act_quant_TOPS"] = round(fused_tops, 2)
        extra["linear_with_dynamic_act_quant_separate_operators_TOPS"] = round(separate_tops, 2)
        extra["linear_m2048_host_buffers_in_and_out"] = bench_linear_from_host(
            L, Q, _C, _ops, r["tensors"], M, K, N, 10)
        del r["tensors"]
        for m in (1, 16):
            # at least 400 launches between the events: the ~50 us from the first event to the
            # first kernel's start would otherwise be a tenth of 50 launches of 7 us
            rs = bench_linear(L, Q, _C, _ops, m, K, N, max(args.steps, 400), args.warmup, seed=3)
            # us / GB/s: average of back-to-back launches between one pair of events (as the
            # headline); the median of individually bracketed launches, event cost included, beside it
            # cold_*: the same launches cycling through weight copies that exceed the last-level
            # cache, i.e. every byte from HBM (the back-to-back figure re-reads one 45 MB matrix,
            # which stays in the 256 MB cache between launches)
            cold_us = bench_linear_cold_weights(L, _C, _ops, rs["tensors"], m, K, N, max(10, args.steps // 2))
            # us / GB/s / frac_of_8TBs: weights from HBM (the cycling copies); *_llc_resident / *_weights_in_llc:
            # the back-to-back launches on one matrix, which is cache bandwidth, not HBM bandwidth
            extra[f"linear_m{m}"] = {"us": round(cold_us, 2),
                                     "GB/s": round(rs["bytes"] / cold_us / 1e3, 1),
                                     "frac_of_8TBs": round(rs["bytes"] / cold_us / 1e3 / PEAK_HBM_GBS, 4),
                                     "us_weights_in_llc": round(rs["avg_kernel_ms"] * 1e3, 2),
                                     "bracketed_launch_median_us": round(rs["median_ms"] * 1e3, 2),
                                     "GB/s_weights_in_llc": round(rs["gbs"], 1),
                                     "frac_of_8TBs_llc_resident": round(rs["gbs"] / PEAK_HBM_GBS, 4),
                                     "TOP/s_weights_in_llc": round(rs["kernel_tops"], 2), "bytes": rs["bytes"]}
            del rs["tensors"]
        # the same layer at a prefill-sized M: more tiles per CU, better-filled rounds
        rl = bench_linear(L, Q, _C, _ops, 8192, K, N, max(10, args.steps // 2), max(3, args.warmup // 2), seed=5)
        extra["linear_m8192"] = {"us": round(rl["avg_kernel_ms"] * 1e3, 2), "TOP/s": round(rl["kernel_tops"], 2),
                                 "frac_of_int8_peak": round(rl["kernel_tops"] / PEAK_INT8_TOPS, 4)}
        del rl["tensors"]
        extra["weight_only_group64_k4096_n11008"] = bench_weight_only(L, _C, args.steps, args.warmup)
        extra["module_breadth"] = bench_breadth(L, Q, _C, args.steps, args.warmup)
        extra["quant_roundtrip_4096x4096x16"] = bench_quant_roundtrip(
            L, Q, _C, max(10, args.steps // 2), max(3, args.warmup // 2))
        extra["dynamic_mlp_784_256_10_batch64"] = bench_dynamic_mlp(L, Q, _C, args.steps, args.warmup)
        extra["vit_b16_linears_batch64"] = bench_vit_linears(L, Q, _C, _ops, max(10, args.steps // 2),
                                                             max(3, args.warmup // 2))
        extra["vit_b16_dynamic_int8_batch64"] = bench_vit_b16(L, _C, max(10, args.steps // 2),
                                                              max(3, args.warmup // 2))
        extra["resnet50_int8_batch32"] = bench_resnet50(L, _C, max(10, args.steps // 2),
                                                        max(3, args.warmup // 2))
        line["extra"] = extra
    if not args.no_cpu_baseline:
        tops, dt, spent, cores, single = cpu_baseline_linear(K, N, args.cpu_sample_rows)
        line["cpu_baseline"] = {
            "value": round(tops, 5),
            "unit": "TOP/s",
            "cores": cores,
            "kind": "port",
            "sample": f"{args.cpu_sample_rows} of {M} rows of the same layer; median of 8 calls, "
                      f"each = per-call weight dequantize + float32 GEMM + bias "
                      f"({dt:.2f} s per call, {spent:.0f} s of CPU time in all)",
            "single_thread": single,
        }
        # the timed outputs against the CPU restatement, in this leg only
        checks = {"linear_m2048_fp16_output": verify_linear_sample(r["verify"])}
        qv = verify_quant_slice()
        if qv is not None:
            checks["quantize_dequantize_per_channel_slice"] = qv
        line["verified"] = all(c["bit_exact"] for c in checks.values())
        line["verification"] = checks
    print(json.dumps(line))
    if line.get("verified") is False:
        print("bench.py: a timed output differs from the CPU restatement", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())

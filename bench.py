#!/usr/bin/env python3
"""Benchmark of the matrix-multiplication path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--all]

A step is one pass of the hot path over one batch of synthetic input: the fp16-input /
fp32-accumulate GEMM at M = N = K = 4096 (configuration 3: y zeros, y += A*B) with the inputs
already resident in HBM, issued the way the operator layer issues it -- a fresh TensorData y
from the buffer pool, Compute::GemmHalf(y, A, B), ResourceManager::Clean() -- which is one
kernel launch per step.  The script does W untimed steps, then times exactly K steps between
two synchronisation points and prints ONE JSON line.  `value` is TFLOP/s of those K steps
(2*4096^3 flop each).  The same line carries

  roofline      the GEMM kernel against the dense fp16 MFMA peak, from HIP events recorded on
                the stream the kernel runs on, with the shader clock polled beside the leg;
  gemm_accumulate_into_used_out_variant   the raw C-ABI call adding into an out that is in use;
  gemm_zero_operands_variant              the headline leg on all-zero operands (clock beside it);
  spmm          the CSR x dense product of configuration 5 (8192 x 8192 at 1 % times
                8192 x 256), timed the same way, against the HBM peak on algorithmic bytes;
  configs       configurations 1, 2 and 4 (fp32 GEMM, batched fp32 GEMM with a shared B, the
                3-layer MLP forward), each with its own roofline object;
  cpu_baseline  the reference's own scalar CPU GEMM (built into oracle/_ref from the
                reference's NaiveGemm.cpp; the plain-C port when that build is absent) timed
                on a bounded slice of the same workload on this machine's host cores.

Everything runs on one GPU; --gpus above 1 is refused.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA, vendor figure
PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E


def recorded_traffic(profile_name):
    """HBM-side bytes per launch from the committed rocprofv3 summary (FETCH_SIZE and
    WRITE_SIZE counter runs, scaled by the copy-kernel calibration); None when absent."""
    path = os.path.join(ROOT, "profiles", profile_name)
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return int(line.split(":")[1].split()[0])
    except OSError:
        pass
    return None


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=10)
    p.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    p.add_argument("--all", action="store_true",
                   help="also time the neighbouring kernels (backward pass, conversions, CSR x "
                        "CSR, one-pass kernels; reported under 'others')")
    p.add_argument("--only", choices=["gemm", "gemm_operator", "spmm", "copy", "backward", "backward_reference", "gemm_f32",
                                      "csr", "spgemm", "shapes", "mfma_ceiling", "one"], default=None,
                   help="run a single kernel (for profiler runs); the JSON line is reduced")
    p.add_argument("--dims", type=int, nargs=3, metavar=("M", "N", "K"), default=[1024, 1024, 1024],
                   help="with --only one: the product to time")
    p.add_argument("--f32", action="store_true",
                   help="with --only one: sph_gemm_f32_ex instead of sph_gemm_f16f32")
    p.add_argument("--flags", type=int, default=0,
                   help="with --only one: SPH_GEMM_* flags of the call (1 overwrite, 2 A stored "
                        "K x M, 4 B stored N x K)")
    p.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                   help="untimed run-up before each timed leg that lets the clock reach its "
                        "working frequency (0 = none)")
    p.add_argument("--zero-operands", action="store_true",
                   help="with --only gemm / gemm_operator: all-zero A and B, to see how far the clock (and the "
                        "rate) depends on operand values; the line says data = zeros")
    return p.parse_args()


# The shader clock idles at ~160 MHz and takes about half a second of load to reach its working
# frequency (rocm-smi polled beside a run: 150 -> 2140 -> 2370 -> 2394 MHz at 0.2 s intervals).
# Every timed leg is therefore preceded by SETTLE_MS of the same launches, untimed and not
# counted as warm-up steps, so that the figure is the sustained one.
SETTLE_MS = 600.0


def settle(capi, launch):
    if SETTLE_MS <= 0:
        return
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(20):
            launch()
        capi.sync()


class ClockSampler:
    """Polls the shader clock (sclk) in a thread beside a leg, so that the line shows at what
    clock a figure was taken.  One visible card with a readable pp_dpm_sclk: that file, every
    20 ms; otherwise `rocm-smi --showclocks` as fast as it returns."""

    def __init__(self):
        import glob
        import threading
        self.samples = []      # (seconds since start, MHz)
        self.source = None
        self._stop = threading.Event()
        self._t0 = time.perf_counter()
        files = [f for f in glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")
                 if os.access(f, os.R_OK)]
        self._file = files[0] if len(files) == 1 else None
        self._thread = threading.Thread(target=self._run, daemon=True)

    @staticmethod
    def _current_from_levels(text):
        # "1: 1679Mhz *": the starred level is the current clock
        for line in text.splitlines():
            if "*" in line:
                digits = "".join(ch if ch.isdigit() else " " for ch in line.split(":", 1)[-1])
                return float(digits.split()[0])
        return None

    def _read(self):
        if self._file is not None:
            try:
                mhz = self._current_from_levels(open(self._file).read())
                if mhz is not None:
                    self.source = "pp_dpm_sclk"
                    time.sleep(0.02)
                    return mhz
            except OSError:
                pass
            self._file = None
        import re
        import subprocess
        try:
            text = subprocess.run(["rocm-smi", "--showclocks"], stdout=subprocess.PIPE,
                                  stderr=subprocess.DEVNULL, text=True, timeout=5).stdout
        except (OSError, subprocess.SubprocessError):
            return None
        best = None
        for line in text.splitlines():
            if "sclk" in line:
                m = re.search(r"\((\d+)\s*Mhz\)", line, re.I)
                if m:
                    best = max(best or 0.0, float(m.group(1)))   # the card under load
        if best is not None:
            self.source = "rocm-smi --showclocks"
        return best

    def _run(self):
        while not self._stop.is_set():
            mhz = self._read()
            if mhz is None:
                if self._file is None and self.source is None:
                    return      # no way to read the clock here
                continue
            self.samples.append((time.perf_counter() - self._t0, mhz))

    def start(self):
        self._thread.start()
        return self

    def stop(self, window_s=0.35):
        """Stops polling; summary of the samples of the last `window_s` seconds of the leg."""
        t_end = time.perf_counter() - self._t0
        self._stop.set()
        self._thread.join(timeout=6)
        mhz = [m for t, m in self.samples if t >= t_end - window_s and t <= t_end]
        if not mhz:
            mhz = [m for _, m in self.samples[-2:]]
        out = {"source": self.source, "samples_mhz": [int(m) for _, m in self.samples][-40:],
               "window_s": window_s}
        if mhz:
            out["sclk_mhz_under_load"] = float(np.median(mhz))
            out["samples_in_window"] = len(mhz)
        return out


def timed_launches(capi, launch, steps, warmup, clock=None):
    """Average milliseconds per launch from HIP events on the launch stream, and the wall-clock
    milliseconds per step between two stream synchronisations.  With `clock` (a dict) the
    shader clock is polled beside the leg and its summary is put there."""
    sampler = ClockSampler().start() if clock is not None else None
    try:
        return _timed_launches(capi, launch, steps, warmup)
    finally:
        if sampler is not None:
            clock.update(sampler.stop())


def _timed_launches(capi, launch, steps, warmup):
    settle(capi, launch)
    for _ in range(warmup):
        launch()
    capi.sync()
    start, stop = capi.Event(), capi.Event()
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        launch()
    stop.record()
    capi.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    event_ms = stop.elapsed_ms_since(start) / steps
    start.destroy()
    stop.destroy()
    return event_ms, wall_ms


def timed_maybe_graph(capi, launch, steps, warmup, graph):
    """Event time per step of `launch`, issued call by call or recorded once and replayed."""
    if not graph:
        return timed_launches(capi, launch, steps, warmup)[0]
    with capi.Graph() as recorded:
        launch()
    event_ms, _ = timed_launches(capi, recorded.launch, steps, warmup)
    recorded.destroy()
    return event_ms


def bench_gemm_f16(capi, synth, steps, warmup, flags=0, zero_operands=False, clock=None):
    n = 4096
    d = synth.config3(n)
    if zero_operands:
        d["A"][...] = 0
        d["B"][...] = 0
    dA = capi.DeviceBuffer.from_array(d["A"])
    dB = capi.DeviceBuffer.from_array(d["B"])
    dC = capi.DeviceBuffer.from_array(d["C"])
    capi.require_gemm_extents(dC, dA, dB, n, n, n, 1, n * n, n * n, n * n, operand_bytes=2)

    def launch():
        capi.call("sph_gemm_f16f32", dC.ptr, dA.ptr, dB.ptr, n, n, n, 1, n * n, n * n, n * n, flags)

    event_ms, wall_ms = timed_launches(capi, launch, steps, warmup, clock=clock)
    for b in (dA, dB, dC):
        b.release()
    return event_ms, wall_ms, d


def bench_gemm_f16_operator(capi, synth, steps, warmup, zero_operands=False, clock=None):
    """Configuration 3 as the operator layer runs it: per step a fresh y [4096, 4096] is taken
    from the buffer pool (it reads as zeros, the fill is deferred), Compute::GemmHalf(y, A, B)
    adds the product to it -- seeing the fresh state, it stores the product instead of filling,
    reading and adding -- and ResourceManager::Clean() hands the step's blocks back.  Driven
    through the C view of the C++ layer that the parity tests use."""
    from tests import host_layer as hl
    n = 4096
    d = synth.config3(n)
    if zero_operands:
        d["A"][...] = 0
        d["B"][...] = 0
    dA = capi.DeviceBuffer.from_array(d["A"])
    dB = capi.DeviceBuffer.from_array(d["B"])
    assert dA.nbytes >= 2 * n * n and dB.nbytes >= 2 * n * n
    sampler = ClockSampler().start() if clock is not None else None
    try:
        event_ms, wall_ms = hl.bench_gemm_half_fresh_y(dA.ptr, dB.ptr, n, steps, warmup, SETTLE_MS)
    finally:
        if sampler is not None:
            clock.update(sampler.stop())
    dA.release()
    dB.release()
    return event_ms, wall_ms, d


def bench_spmm(capi, synth, steps, warmup):
    d = synth.config5()
    M, K, N = d["M"], d["K"], d["N"]
    dV = capi.DeviceBuffer.from_array(d["V"])
    dCol = capi.DeviceBuffer.from_array(d["COL"])
    dRow = capi.DeviceBuffer.from_array(d["ROW"])
    dB = capi.DeviceBuffer.from_array(d["B"])
    dC = capi.DeviceBuffer.from_array(d["C"])
    capi.require_csr_extents(dC, dV, dCol, dRow, dB, M, K, N, int(d["V"].size))
    capi.validate_csr(dCol, dRow, M, K, int(d["V"].size))

    def launch():
        capi.call("sph_spmm_csr_f32", dC.ptr, dV.ptr, dCol.ptr, dRow.ptr, M, K, N, dB.ptr, 0)

    event_ms, wall_ms = timed_launches(capi, launch, steps, warmup)
    for b in (dV, dCol, dRow, dB, dC):
        b.release()
    nnz = int(d["V"].size)
    # store mode: V + COL, ROW, B once, out written once
    alg_bytes = nnz * 8 + (M + 1) * 4 + K * N * 4 + M * N * 4
    return event_ms, wall_ms, d, nnz, alg_bytes


def bench_f32(capi, A, B, C, M, N, K, batch, sb, steps, warmup):
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, C))
    capi.require_gemm_extents(dC, dA, dB, M, N, K, batch, M * N, M * K, sb)

    def launch():
        capi.call("sph_gemm_f32", dC.ptr, dA.ptr, dB.ptr, M, N, K, batch, M * N, M * K, sb)

    event_ms, _ = timed_launches(capi, launch, steps, warmup)
    for b in (dA, dB, dC):
        b.release()
    return event_ms


def bench_mlp(capi, synth, steps, warmup, fused=False, graph=False):
    """Configuration 4 through the C ABI: per layer ones[batch,1] x bias (K = 1 GEMM), x x W,
    ReLU between layers -- the call sequence of Linear's forward pass; with `fused` one
    sph_linear_forward_f32 per layer instead (same result bits)."""
    d = synth.config4()
    batch = d["x"].shape[0]
    sizes = [d["x"].shape[1]] + [w.shape[1] for w in d["W"]]
    x = capi.DeviceBuffer.from_array(d["x"])
    W = [capi.DeviceBuffer.from_array(w) for w in d["W"]]
    b = [capi.DeviceBuffer.from_array(v) for v in d["b"]]
    ones = capi.DeviceBuffer.from_array(np.ones(batch, np.float32))
    y = [capi.DeviceBuffer(4 * batch * n) for n in sizes[1:]]
    act = [capi.DeviceBuffer(4 * batch * n) for n in sizes[1:-1]]

    def launch():
        cur = x
        for l in range(3):
            n_in, n_out = sizes[l], sizes[l + 1]
            if fused:
                capi.call("sph_linear_forward_f32", y[l].ptr, cur.ptr, W[l].ptr, b[l].ptr, batch,
                          n_in, n_out, capi.SPH_LINEAR_RELU if l < 2 else 0)
                cur = y[l]
                continue
            capi.call("sph_fill_f32", y[l].ptr, 0.0, batch * n_out)
            capi.call("sph_gemm_f32", y[l].ptr, ones.ptr, b[l].ptr, batch, n_out, 1, 1,
                      batch * n_out, batch, n_out)
            capi.call("sph_gemm_f32", y[l].ptr, cur.ptr, W[l].ptr, batch, n_out, n_in, 1,
                      batch * n_out, batch * n_in, n_in * n_out)
            if l < 2:
                capi.call("sph_relu_f32", act[l].ptr, y[l].ptr, batch * n_out)
                cur = act[l]

    event_ms = timed_maybe_graph(capi, launch, steps, warmup, graph)
    for buf in [x, ones] + W + b + y + act:
        buf.release()
    flops = 2.0 * batch * sum(sizes[l] * sizes[l + 1] for l in range(3))
    return event_ms, flops


def bench_mlp_backward(capi, synth, steps, warmup, direct, graph=False, fused_update=False):
    """Backward pass + SGD update of configuration 4's three Linear layers through the C ABI
    (the call sequence of LinearBackProp::m_runBackProp per layer, ReLUBackward between
    layers).  direct=False materialises the transposes, zero-fills and uses Scale + Sub like
    the reference; direct=True uses the transposed-read / overwrite flags and the one-pass SGD
    step; fused_update (with direct) ends the weight and bias gradient products in the update
    itself (sph_gemm_f32_sgd), so neither gradient is stored.  Parameters drift over the steps;
    only time is taken here."""
    d = synth.config4()
    batch = d["x"].shape[0]
    sizes = [d["x"].shape[1]] + [w.shape[1] for w in d["W"]]
    lr = 1e-6
    W = [capi.DeviceBuffer.from_array(w) for w in d["W"]]
    b = [capi.DeviceBuffer.from_array(v) for v in d["b"]]
    acts = [capi.DeviceBuffer.from_array(synth.uniform(400 + l, (batch, sizes[l])))
            for l in range(3)]                                   # layer inputs x_l
    pre = [capi.DeviceBuffer.from_array(synth.uniform(410 + l, (batch, sizes[l + 1])))
           for l in range(2)]                                    # pre-activations of layers 0, 1
    dy_top = capi.DeviceBuffer.from_array(synth.uniform(420, (batch, sizes[3])))
    grads = [capi.DeviceBuffer(4 * batch * n) for n in sizes]   # d(x_l), and scratch d(pre)
    dpre = [capi.DeviceBuffer(4 * batch * n) for n in sizes[1:3]]
    big = max(sizes[l] * sizes[l + 1] for l in range(3))
    wt = capi.DeviceBuffer(4 * big)
    xt = capi.DeviceBuffer(4 * batch * max(sizes))
    dw = capi.DeviceBuffer(4 * big)
    temp = capi.DeviceBuffer(4 * big)
    ones = capi.DeviceBuffer.from_array(np.ones(batch, np.float32))
    dB = capi.DeviceBuffer(4 * max(sizes))
    TA, TB, OV = capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B, capi.SPH_GEMM_OVERWRITE

    def sgd(z, dz, count):
        if direct:
            capi.call("sph_sgd_step_f32", z.ptr, dz.ptr, lr, count)
        else:
            capi.call("sph_scale_f32", temp.ptr, dz.ptr, lr, count)
            capi.call("sph_sub_f32", z.ptr, z.ptr, temp.ptr, count, 0, 0, 0)

    def layer(l, dy):
        n_in, n_out = sizes[l], sizes[l + 1]
        dx, x = grads[l], acts[l]
        capi.call("sph_fill_f32", dx.ptr, 0.0, batch * n_in)       # a fresh dx tensor
        if direct:
            capi.call("sph_gemm_f32_ex", dx.ptr, dy.ptr, W[l].ptr, batch, n_in, n_out, 1,
                      batch * n_in, batch * n_out, n_in * n_out, TB)
            if fused_update:
                capi.call("sph_gemm_f32_sgd", W[l].ptr, x.ptr, dy.ptr, n_in, n_out, batch, 1.0, lr,
                          TA)
                capi.call("sph_gemm_f32_sgd", b[l].ptr, ones.ptr, dy.ptr, 1, n_out, batch,
                          1.0 / batch, lr, 0)
                return
            capi.call("sph_gemm_f32_ex", dw.ptr, x.ptr, dy.ptr, n_in, n_out, batch, 1,
                      n_in * n_out, n_in * batch, batch * n_out, TA | OV)
        else:
            capi.call("sph_transpose_f32", wt.ptr, W[l].ptr, n_in, n_out, 1, 0)
            capi.call("sph_gemm_f32", dx.ptr, dy.ptr, wt.ptr, batch, n_in, n_out, 1,
                      batch * n_in, batch * n_out, n_in * n_out)
            capi.call("sph_transpose_f32", xt.ptr, x.ptr, batch, n_in, 1, 0)
            capi.call("sph_fill_f32", dw.ptr, 0.0, n_in * n_out)
            capi.call("sph_gemm_f32", dw.ptr, xt.ptr, dy.ptr, n_in, n_out, batch, 1,
                      n_in * n_out, n_in * batch, batch * n_out)
        sgd(W[l], dw, n_in * n_out)
        if direct:
            capi.call("sph_gemm_f32_ex", dB.ptr, ones.ptr, dy.ptr, 1, n_out, batch, 1, n_out,
                      batch, batch * n_out, OV)
        else:
            capi.call("sph_fill_f32", ones.ptr, 1.0, batch)
            capi.call("sph_fill_f32", dB.ptr, 0.0, n_out)
            capi.call("sph_gemm_f32", dB.ptr, ones.ptr, dy.ptr, 1, n_out, batch, 1, n_out,
                      batch, batch * n_out)
        capi.call("sph_scale_f32", dB.ptr, dB.ptr, 1.0 / batch, n_out)
        sgd(b[l], dB, n_out)

    def launch():
        dy = dy_top
        for l in (2, 1, 0):
            layer(l, dy)
            if l > 0:
                capi.call("sph_fill_f32", dpre[l - 1].ptr, 0.0, batch * sizes[l])
                capi.call("sph_relu_backward_f32", dpre[l - 1].ptr, grads[l].ptr, pre[l - 1].ptr,
                          batch * sizes[l])
                dy = dpre[l - 1]

    event_ms = timed_maybe_graph(capi, launch, steps, warmup, graph)
    for buf in W + b + acts + pre + grads + dpre + [dy_top, wt, xt, dw, temp, ones, dB]:
        buf.release()
    flops = 2.0 * 2.0 * batch * sum(sizes[l] * sizes[l + 1] for l in range(3))
    return event_ms, flops


# Shapes off the kernels' natural grid: a K that is no multiple of the K step, an N (or M) that is
# no multiple of the copy width, operands stored the other way round.
# small products (few output tiles: a layer of a small network on a small batch) ride along
SMALL = [(256, 1024, 1024), (100, 1024, 784), (1024, 10, 1024), (128, 128, 4096), (512, 1024, 1024)]
OFF_GRID_F16 = [(4096, 4096, 4096), (4096, 4096, 4080), (4096, 4096, 4095), (4096, 4100, 4096),
                (4096, 4095, 4096), (4095, 4095, 4095), (2048, 2052, 2048), (1024, 1024, 1001),
                (1024, 1024, 1024), (1024, 1024, 4096), (2048, 2048, 2048), (3072, 2048, 2048),
                (2048, 4096, 2048), (1025, 1025, 1025), (1001, 1001, 1001), (4097, 4097, 4097),
                (128, 128, 4095)] + SMALL
OFF_GRID_F32 = [(1024, 1024, 1024), (1024, 1024, 1000), (1024, 1024, 1001), (1000, 1000, 1000),
                (1001, 1001, 1001), (1024, 1026, 1024), (2048, 2048, 2047), (2048, 2050, 2048),
                (4096, 4096, 4096), (4096, 4095, 4096), (4096, 4096, 4100), (1025, 1025, 1025),
                (8192, 65, 64), (384, 1024, 1024)] + SMALL


def bench_off_grid(capi, synth, steps, warmup):
    """Event time per launch of one M x N x K product per shape and storage flag set."""
    rows = []

    def one(entry, M, N, K, flags, A, B):
        C = np.zeros((M, N), np.float32)
        dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, C))
        capi.require_gemm_extents(dC, dA, dB, M, N, K, 1, M * N, M * K, K * N,
                                  operand_bytes=2 if entry == "sph_gemm_f16f32" else 4)

        def launch():
            capi.call(entry, dC.ptr, dA.ptr, dB.ptr, M, N, K, 1, M * N, M * K, K * N, flags)

        ms, _ = timed_launches(capi, launch, steps, warmup)
        for d in (dA, dB, dC):
            d.release()
        rows.append({"entry_point": entry, "M": M, "N": N, "K": K, "flags": flags,
                     "launch_ms": ms, "tflops": 2.0 * M * N * K / (ms * 1e-3) / 1e12})

    for M, N, K in OFF_GRID_F16:
        A = synth.normal(1, (M, K), 1.0 / np.sqrt(K)).astype(np.float16)
        B = synth.normal(2, (K, N), 1.0 / np.sqrt(K)).astype(np.float16)
        for flags in (0, capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B):
            # the values only have to be typical; the buffers are read with the other pitch
            one("sph_gemm_f16f32", M, N, K, flags, A, B)
    for M, N, K in OFF_GRID_F32:
        A = synth.uniform(1, (M, K))
        B = synth.uniform(2, (K, N))
        for flags in (0, capi.SPH_GEMM_TRANS_A, capi.SPH_GEMM_TRANS_B):
            one("sph_gemm_f32_ex", M, N, K, flags, A, B)
    return rows


def bench_one(capi, synth, M, N, K, f32, flags, steps, warmup):
    """One M x N x K product (operands as for --only shapes), for profiler runs of one kernel."""
    entry = "sph_gemm_f32_ex" if f32 else "sph_gemm_f16f32"
    if f32:
        A, B = synth.uniform(1, (M, K)), synth.uniform(2, (K, N))
    else:
        A = synth.normal(1, (M, K), 1.0 / np.sqrt(K)).astype(np.float16)
        B = synth.normal(2, (K, N), 1.0 / np.sqrt(K)).astype(np.float16)
    C = np.zeros((M, N), np.float32)
    dA, dB, dC = (capi.DeviceBuffer.from_array(x) for x in (A, B, C))
    capi.require_gemm_extents(dC, dA, dB, M, N, K, 1, M * N, M * K, K * N,
                              operand_bytes=4 if f32 else 2)

    def launch():
        capi.call(entry, dC.ptr, dA.ptr, dB.ptr, M, N, K, 1, M * N, M * K, K * N, flags)

    ms, _ = timed_launches(capi, launch, steps, warmup)
    for d in (dA, dB, dC):
        d.release()
    tf = 2.0 * M * N * K / (ms * 1e-3) / 1e12
    return {"entry_point": entry, "M": M, "N": N, "K": K, "flags": flags, "launch_ms": ms,
            "tflops": tf, "frac_of_peak": tf / (PEAK_FP32_TFLOPS if f32 else PEAK_FP16_TFLOPS)}


def bench_sgd_step(capi, steps, warmup, mib=64):
    """One-pass SGD update over `mib` MiB of parameters: reads z and dz, writes z."""
    n = mib * (1 << 20) // 4
    z = capi.DeviceBuffer.from_array(np.ones(n, np.float32))
    dz = capi.DeviceBuffer.from_array(np.ones(n, np.float32))

    def launch():
        capi.call("sph_sgd_step_f32", z.ptr, dz.ptr, 1e-6, n)

    event_ms, _ = timed_launches(capi, launch, steps, warmup)
    z.release()
    dz.release()
    return event_ms, 3 * 4 * n


def bench_csr_conversion(capi, synth, steps, warmup):
    """Dense -> CSR (row offsets + fill, no host read-back of nnz inside the timed region) and
    CSR -> dense on configuration 5's matrix (8192 x 8192 fp32 at 1 %)."""
    d = synth.config5()
    M, K = d["M"], d["K"]
    nnz = int(d["V"].size)
    dense = capi.DeviceBuffer.from_array(synth.densify(d["V"], d["COL"], d["ROW"], M, K))
    row = capi.DeviceBuffer(4 * (M + 1))
    val = capi.DeviceBuffer(4 * nnz)
    col = capi.DeviceBuffer(4 * nnz)

    def to_csr():
        capi.call("sph_csr_row_offsets_f32", row.ptr, dense.ptr, M, K, K, None)
        capi.call("sph_csr_fill_f32", val.ptr, col.ptr, row.ptr, dense.ptr, M, K, K)

    def to_csr_one_call():
        capi.call("sph_csr_from_dense_f32", val.ptr, col.ptr, row.ptr, nnz, dense.ptr, M, K, K,
                  None)

    def to_dense():
        capi.call("sph_csr_to_dense_f32", dense.ptr, K, val.ptr, col.ptr, row.ptr, M, K)

    ms_csr, _ = timed_launches(capi, to_csr, steps, warmup)
    ms_one, _ = timed_launches(capi, to_csr_one_call, steps, warmup)
    ms_dense, _ = timed_launches(capi, to_dense, steps, warmup)
    for b in (dense, row, val, col):
        b.release()
    dense_bytes = 4 * M * K
    csr_bytes = 8 * nnz + 4 * (M + 1)
    return ms_csr, ms_one, ms_dense, dense_bytes, csr_bytes


def bench_spgemm(capi, synth, steps, warmup, n=8192, per_row=8.0):
    """CSR x CSR -> CSR of two n x n matrices with `per_row` entries per row on average: the
    counting pass (row offsets, no host read-back inside the timed region) and the fill pass."""
    a = synth.csr_matrix(7001, n, n, per_row)
    b = synth.csr_matrix(7002, n, n, per_row)
    bufs = [capi.DeviceBuffer.from_array(x) for x in a + b]
    row = capi.DeviceBuffer(4 * (n + 1))
    import ctypes
    nnz = ctypes.c_uint32(0)
    ptrs = [x.ptr for x in bufs]
    capi.call("sph_spgemm_row_offsets_f32", row.ptr, *ptrs, n, n, n, ctypes.byref(nnz))
    val = capi.DeviceBuffer(4 * max(nnz.value, 1))
    col = capi.DeviceBuffer(4 * max(nnz.value, 1))

    def launch():
        capi.call("sph_spgemm_row_offsets_f32", row.ptr, *ptrs, n, n, n, None)
        capi.call("sph_spgemm_fill_f32", val.ptr, col.ptr, row.ptr, *ptrs, n, n, n)

    def one_call():
        capi.call("sph_spgemm_f32", val.ptr, col.ptr, row.ptr, max(nnz.value, 1), *ptrs, n, n, n,
                  None)

    event_ms, _ = timed_launches(capi, launch, steps, warmup)
    one_call_ms, _ = timed_launches(capi, one_call, steps, warmup)
    for x in bufs + [row, val, col]:
        x.release()
    # products: for every entry of A, the length of the matching row of B
    lengths = np.diff(b[2].astype(np.int64))
    products = int(lengths[a[1]].sum())
    nbytes = 8 * (a[0].size + b[0].size + nnz.value) + 3 * 4 * (n + 1)
    return event_ms, products, nnz.value, nbytes, a[0].size, b[0].size, one_call_ms


def bench_sparse_linear(capi, synth, steps, warmup, batch=256):
    """Forward of a Linear layer whose weight is configuration 5's matrix kept as CSR
    (8192 inputs, 8192 outputs, 1 % of the weights), batch 256, issued as the C++ layer's
    NN::SparseLinearForward issues it: x transposed, ones, zero fill, bias x ones (K = 1 GEMM),
    CSR x dense accumulating, result transposed back.  Returns the milliseconds per forward and
    of the CSR x dense launch alone."""
    d = synth.config5()
    outs, ins = d["M"], d["K"]
    x = capi.DeviceBuffer.from_array(synth.uniform(6100, (batch, ins)))
    bias = capi.DeviceBuffer.from_array(synth.uniform(6101, (outs,), -0.1, 0.1))
    dV, dCol, dRow = (capi.DeviceBuffer.from_array(d[k]) for k in ("V", "COL", "ROW"))
    xT = capi.DeviceBuffer(4 * ins * batch)
    yT = capi.DeviceBuffer(4 * outs * batch)
    y = capi.DeviceBuffer(4 * outs * batch)
    ones = capi.DeviceBuffer(4 * batch)

    def product():
        capi.call("sph_spmm_csr_f32", yT.ptr, dV.ptr, dCol.ptr, dRow.ptr, outs, ins, batch, xT.ptr, 1)

    def forward_unfused():
        capi.call("sph_transpose_f32", xT.ptr, x.ptr, batch, ins, 1, 0)
        capi.call("sph_fill_f32", ones.ptr, 1.0, batch)
        capi.call("sph_fill_f32", yT.ptr, 0.0, outs * batch)
        capi.call("sph_gemm_f32", yT.ptr, bias.ptr, ones.ptr, outs, batch, 1, 1, outs * batch, outs,
                  batch)
        product()
        capi.call("sph_transpose_f32", y.ptr, yT.ptr, outs, batch, 1, 0)

    def forward():
        capi.call("sph_transpose_f32", xT.ptr, x.ptr, batch, ins, 1, 0)
        capi.call("sph_spmm_csr_bias_f32", yT.ptr, dV.ptr, dCol.ptr, dRow.ptr, outs, ins, batch,
                  xT.ptr, bias.ptr)
        capi.call("sph_transpose_f32", y.ptr, yT.ptr, outs, batch, 1, 0)

    ms, _ = timed_launches(capi, forward, steps, warmup)
    ms_unfused, _ = timed_launches(capi, forward_unfused, steps, warmup)
    ms_product, _ = timed_launches(capi, product, steps, warmup)
    for b in (x, bias, dV, dCol, dRow, xT, yT, y, ones):
        b.release()
    return ms, ms_product, int(d["V"].size), ms_unfused


def bench_allocation(capi, nbytes=64 << 20, rounds=200):
    """Host-side cost of taking and returning one device block of `nbytes`: the blocking pair
    (hipMalloc / hipFree) against the stream-ordered pair the buffer pool uses on a miss."""
    import ctypes
    out = {}
    for name, take, give in (("malloc_free", "sph_malloc", "sph_free"),
                             ("malloc_async_free_async", "sph_malloc_async", "sph_free_async")):
        ptr = ctypes.c_void_p()
        for _ in range(5):
            capi.call(take, ctypes.byref(ptr), nbytes)
            capi.call(give, ptr)
        capi.sync()
        t0 = time.perf_counter()
        for _ in range(rounds):
            capi.call(take, ctypes.byref(ptr), nbytes)
            capi.call(give, ptr)
        capi.sync()
        out[name + "_us"] = (time.perf_counter() - t0) * 1e6 / rounds
    out["block_bytes"] = nbytes
    return out


def bench_elementwise(capi, steps, warmup, n=4096):
    """The one-pass kernels over n x n floats (64 MiB at n = 4096): algorithmic GB/s each."""
    count = n * n
    x = capi.DeviceBuffer.from_array(np.ones((n, n), np.float32))
    z = capi.DeviceBuffer.from_array(np.ones((n, n), np.float32))
    y = capi.DeviceBuffer(4 * count)
    half = capi.DeviceBuffer(2 * count)
    runs = [
        ("transpose", lambda: capi.call("sph_transpose_f32", y.ptr, x.ptr, n, n, 1, 0), 8),
        ("relu", lambda: capi.call("sph_relu_f32", y.ptr, x.ptr, count), 8),
        ("relu_backward", lambda: capi.call("sph_relu_backward_f32", y.ptr, x.ptr, z.ptr, count), 16),
        ("scale", lambda: capi.call("sph_scale_f32", y.ptr, x.ptr, 2.0, count), 8),
        ("sub", lambda: capi.call("sph_sub_f32", y.ptr, x.ptr, z.ptr, count, 0, 0, 0), 12),
        ("sgd_step", lambda: capi.call("sph_sgd_step_f32", y.ptr, x.ptr, 1e-6, count), 12),
        ("fill", lambda: capi.call("sph_fill_f32", y.ptr, 0.0, count), 4),
        ("convert_f32_to_f16", lambda: capi.call("sph_convert_f32_to_f16", half.ptr, x.ptr, count), 6),
    ]
    out = {}
    for name, fn, bytes_per_element in runs:
        ms, _ = timed_launches(capi, fn, steps, warmup)
        gbs = bytes_per_element * count / (ms * 1e-3) / 1e9
        out[name] = {"launch_ms": ms, "gbs": gbs, "frac_hbm_peak": gbs / PEAK_HBM_GBS}
    for b in (x, z, y, half):
        b.release()
    return out


def bench_copy(capi, steps, warmup, mib=64):
    """A plain one-pass kernel of known size (ReLU over `mib` MiB: reads it once, writes it
    once), used to calibrate the profiler's FETCH_SIZE / WRITE_SIZE counters."""
    n = mib * (1 << 20) // 4
    src = capi.DeviceBuffer.from_array(np.ones(n, np.float32))
    dst = capi.DeviceBuffer(4 * n)

    def launch():
        capi.call("sph_relu_f32", dst.ptr, src.ptr, n)

    event_ms, _ = timed_launches(capi, launch, steps, warmup)
    src.release()
    dst.release()
    return event_ms, 4 * n


MFMA_CEILING_VARIANTS = [
    "v_mfma_f32_32x32x16_f16 fed from LDS (12 fragment reads per 16 MFMAs)",
    "v_mfma_f32_16x16x32_f16 fed from LDS (12 fragment reads per 32 MFMAs)",
    "32x32x16 + one workgroup barrier per half step",
    "32x32x16 + 32 KiB per K step of global_load_lds from L2",
    "32x32x16, 8 fragment reads per 16 MFMAs (ratio of a 128 x 128 wavefront part)",
    "16x16x32 + 32 KiB per K step of global_load_lds from L2",
]


def bench_mfma_ceiling(settle_ms, timed):
    """What the matrix cores deliver on N(0, 1/64) operands and on zeros with the 256-tile
    kernel's loop stripped to its parts (sapphire_amd/probe/mfma_ceiling.hip): every variant
    issues the matrix instructions of a 4096^3 product from 256 workgroups of 8 wavefronts."""
    import ctypes
    path = os.path.join(ROOT, "sapphire_amd", "libsapphire_probe.so")
    if not os.path.exists(path):
        raise RuntimeError("%s is missing: build it with `python -m sapphire_amd.build probe`" % path)
    probe = ctypes.CDLL(path)
    probe.sph_probe_flop_per_launch.restype = ctypes.c_double
    probe.sph_probe_mfma_run.argtypes = [ctypes.c_int, ctypes.c_double, ctypes.c_double,
                                         ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    flop = probe.sph_probe_flop_per_launch()
    rows = []
    for variant in range(probe.sph_probe_variants()):
        row = {"variant": variant, "loop": MFMA_CEILING_VARIANTS[variant]}
        for tag, sigma in (("normal_1_64", 1.0 / 64), ("zeros", 0.0)):
            us = ctypes.c_double(0)
            sampler = ClockSampler().start()
            rc = probe.sph_probe_mfma_run(variant, sigma, settle_ms, timed, ctypes.byref(us))
            clock = sampler.stop()
            if rc != 0:
                raise RuntimeError("sph_probe_mfma_run(%d) failed with hipError %d" % (variant, rc))
            row[tag] = {"us_per_launch": us.value, "tflops": flop / (us.value * 1e-6) / 1e12,
                        "sclk_mhz_under_load": clock.get("sclk_mhz_under_load")}
        rows.append(row)
    return {"flop_per_launch": flop, "settle_ms": settle_ms, "timed_launches": timed, "rows": rows}


def f32_roofline(workload, entry, kernel, ms, flops, alg_bytes):
    tf = flops / (ms * 1e-3) / 1e12
    return {"workload": workload, "entry_point": entry, "launch_ms": ms, "value": tf,
            "unit": "TFLOP/s",
            "roofline": {"bound": "mfma", "kernel": kernel, "achieved": tf,
                         "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                         "frac": tf / PEAK_FP32_TFLOPS, "flop_per_step": flops,
                         "algorithmic_bytes_per_step": alg_bytes,
                         "hbm_gbs_on_algorithmic_bytes": alg_bytes / (ms * 1e-3) / 1e9}}


def spmm_gather_path(nnz, n, launch_ms, info):
    """The bound the CSR x dense kernel actually runs against.  Every stored entry gathers one
    row of B (n floats), far more bytes than the algorithmic ones, and they come from L2, not
    HBM: bytes gathered per second, and the L2 requests they take against the rate at which the
    L2 can look requests up (128 channels, one 128-byte line request per channel and clock)."""
    gathered = nnz * n * 4
    line_requests = gathered // 128            # minimum: every 128-byte line asked for once
    channels = 128
    clock_hz = info.clockMHz * 1e6
    ceiling_requests_per_s = channels * clock_hz
    floor_ms = line_requests / ceiling_requests_per_s * 1e3
    return {"gathered_bytes_per_launch": gathered,
            "gathered_tb_per_s": gathered / (launch_ms * 1e-3) / 1e12,
            "min_l2_line_requests_per_launch": line_requests,
            "l2_request_ceiling_per_s": ceiling_requests_per_s,
            "l2_request_ceiling_note": "%d L2 channels x one tag look-up per clock x %d MHz"
                                       % (channels, info.clockMHz),
            "launch_ms_at_l2_request_ceiling": floor_ms,
            "frac_of_l2_request_ceiling": floor_ms / launch_ms}


def cpu_gemm_baseline(d, rows=32):
    """The reference's scalar loop on rows [0, rows) of configuration 3 (inputs widened to fp32
    exactly), one thread, as the reference runs it."""
    from oracle import pyoracle as po
    n = d["A"].shape[0]
    A = np.ascontiguousarray(d["A"][:rows].astype(np.float32))
    B = d["B"].astype(np.float32)
    out = np.zeros((rows, n), np.float32)
    if po.have_ref():
        fn, kind = po.ref().ref_naive_gemm, "reference"
    else:
        fn, kind = po.oracle().orc_naive_gemm, "port"
    t0 = time.perf_counter()
    fn(out.size, po._f(out), po._f(A), po._f(B), rows, n, n)
    dt = time.perf_counter() - t0
    flops = 2.0 * rows * n * n
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": kind,
        "sample": "rows 0..%d of configuration 3 (%dx%dx%d fp32 after exact widening), "
                  "Dense::Naive::Gemm scalar loop, %.1f s" % (rows - 1, rows, n, n, dt),
        "host_cores_available": os.cpu_count(),
    }


def cpu_gemm_all_cores(d):
    """The same per-element arithmetic (k ascending, unfused, bit-identical output) on the whole
    of configuration 3, rows split over the host's cores and B walked with unit stride."""
    from oracle import pyoracle as po
    n = d["A"].shape[0]
    A = d["A"].astype(np.float32)
    B = d["B"].astype(np.float32)
    out = np.zeros((n, n), np.float32)
    threads = max(1, min(os.cpu_count() or 1, 16))
    t0 = time.perf_counter()
    po.gemm_rows(out, A, B, n, n, n, threads=threads)
    dt = time.perf_counter() - t0
    return {"value": 2.0 * n ** 3 / dt / 1e12, "unit": "TFLOP/s", "cores": threads,
            "kind": "port",
            "sample": "whole configuration 3, row-accumulator form of the reference loop "
                      "(bit-identical results), %.1f s" % dt}


def cpu_spmm_baseline(d):
    from oracle import pyoracle as po
    out = np.zeros((d["M"], d["N"]), np.float32)
    t0 = time.perf_counter()
    po.spmm_csr(out, d["V"], d["COL"], d["ROW"], d["M"], d["N"], d["B"], threads=1)
    dt = time.perf_counter() - t0
    return dt


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU; --gpus %d is not supported (the path shards without "
              "collectives and every box here has one GPU)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    global SETTLE_MS
    SETTLE_MS = args.settle_ms
    from sapphire_amd import capi, synth
    capi.call("sph_set_device", 0)
    info = capi.device_info(0)
    device_peak = info.computeUnits * 4096 * info.clockMHz * 1e6 / 1e12  # fp16 flop/clk/CU = 4096

    result = {}
    n = 4096
    flops = 2.0 * n ** 3
    if args.only in (None, "gemm", "gemm_operator"):
        zeros = args.zero_operands and args.only is not None
        operator_leg = args.only in (None, "gemm_operator")
        clock = {}
        leg = bench_gemm_f16_operator if operator_leg else bench_gemm_f16
        event_ms, wall_ms, d3 = leg(capi, synth, args.steps, args.warmup, zero_operands=zeros,
                                    clock=clock)
        tflops = flops / (wall_ms * 1e-3) / 1e12
        kernel_tflops = flops / (event_ms * 1e-3) / 1e12
        if operator_leg:
            entry = ("Compute::GemmHalf(y, A, B) on a fresh TensorData y (accumulate contract "
                     "y += A*B; the operator sees that y's zero fill is still deferred and runs "
                     "sph_gemm_f16f32 with SPH_GEMM_OVERWRITE), ResourceManager::Clean() per step")
            alg_bytes = 2 * 64 * (1 << 20)    # A, B read, y written; the zeros are never read
            profile = "gemm_f16_tile256_config3_fresh_y.txt"
        else:
            entry = "sph_gemm_f16f32 (accumulate into a given out)"
            alg_bytes = 3 * 64 * (1 << 20)
            profile = "gemm_f16_tile256_config3.txt"
        result.update({
            "metric": "GEMM TFLOP/s + % MFMA peak (4096^3 fp16->fp32); SpMM GB/s + % HBM peak",
            "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "settle_ms": args.settle_ms, "ms_per_step": wall_ms,
            "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16 in / f32 accumulate",
            "data": "zeros" if zeros else "synthetic",
            "config": {"workload": "configuration 3: y[4096,4096] f32 (zeros) += A[4096,4096] f16 * "
                                   "B[4096,4096] f16, N(0,1/sqrt(K)) inputs, row-major, one launch "
                                   "per step, inputs resident in HBM",
                       "entry_point": entry},
            "roofline": {"bound": "mfma", "kernel": "GemmF16Tile256",
                         "achieved": kernel_tflops, "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                         "frac": kernel_tflops / PEAK_FP16_TFLOPS,
                         "traffic": recorded_traffic(profile),
                         "traffic_unit": "bytes per launch (profiles/%s)" % profile,
                         "algorithmic_bytes_per_launch": alg_bytes,
                         "launch_ms": event_ms, "flop_per_launch": flops,
                         "peak_from_device": device_peak,
                         "peak_from_device_note": "%d CUs x 4096 flop/clk x %d MHz"
                                                  % (info.computeUnits, info.clockMHz),
                         "clock": clock},
            "device": {"name": info.name.decode(), "arch": info.arch.decode(),
                       "compute_units": info.computeUnits, "clock_mhz": info.clockMHz},
        })
        if args.only is None:
            ev_acc, _, _ = bench_gemm_f16(capi, synth, args.steps, args.warmup)
            result["gemm_accumulate_into_used_out_variant"] = {
                "note": "sph_gemm_f16f32 through the C ABI adding into an out that holds earlier "
                        "results (out is read inside the K loop and written): what a caller "
                        "pays when y is not fresh",
                "launch_ms": ev_acc, "tflops": flops / (ev_acc * 1e-3) / 1e12,
                "frac": flops / (ev_acc * 1e-3) / 1e12 / PEAK_FP16_TFLOPS}
            zclock = {}
            ev_zero, _, _ = bench_gemm_f16_operator(capi, synth, args.steps, args.warmup,
                                                    zero_operands=True, clock=zclock)
            tf_zero = flops / (ev_zero * 1e-3) / 1e12
            result["gemm_zero_operands_variant"] = {
                "note": "the headline leg again (same call, same kernel, same instruction "
                        "stream) on all-zero A and B: the chip holds a power limit, and on "
                        "operands that do not toggle the matrix cores it keeps its full clock; "
                        "compare clock.sclk_mhz_under_load here with roofline.clock",
                "data": "zeros", "launch_ms": ev_zero, "tflops": tf_zero,
                "frac": tf_zero / PEAK_FP16_TFLOPS, "clock": zclock}
            mhz, zmhz = clock.get("sclk_mhz_under_load"), zclock.get("sclk_mhz_under_load")
            if mhz and zmhz:
                result["roofline"]["frac_of_peak_at_measured_clock"] = kernel_tflops / (
                    info.computeUnits * 4096 * mhz * 1e6 / 1e12)
                result["gemm_zero_operands_variant"]["frac_of_peak_at_measured_clock"] = tf_zero / (
                    info.computeUnits * 4096 * zmhz * 1e6 / 1e12)

    if args.only == "mfma_ceiling":
        result["mfma_ceiling"] = bench_mfma_ceiling(args.settle_ms, max(args.steps, 100))

    if args.only == "copy":
        ms, nbytes = bench_copy(capi, args.steps, args.warmup)
        result["copy"] = {"kernel": "ReluKernel", "bytes_read": nbytes, "bytes_written": nbytes,
                          "launch_ms": ms, "gbs": 2 * nbytes / (ms * 1e-3) / 1e9}

    if args.only in ("backward", "backward_reference"):
        ms, fl = bench_mlp_backward(capi, synth, args.steps, args.warmup,
                                    direct=args.only == "backward")
        result["backward"] = {"sequence": "direct" if args.only == "backward" else "reference",
                              "step_ms": ms, "tflops": fl / (ms * 1e-3) / 1e12}

    if args.only == "gemm_f32":
        c2 = synth.config2()
        ms = bench_f32(capi, c2["A"], c2["B"], c2["C"], 512, 512, 512, 16, 0, args.steps,
                       args.warmup)
        tf = 16 * 2 * 512 ** 3 / (ms * 1e-3) / 1e12
        result["gemm_f32"] = {"workload": "configuration 2: A[16,512,512] x B[1,512,512] fp32",
                              "launch_ms": ms, "tflops": tf,
                              "frac_fp32_mfma_peak": tf / PEAK_FP32_TFLOPS}

    if args.only == "shapes":
        result["off_grid_shapes"] = bench_off_grid(capi, synth, min(args.steps, 20), 3)

    if args.only == "one":
        M, N, K = args.dims
        result["one"] = bench_one(capi, synth, M, N, K, args.f32, args.flags, args.steps,
                                  args.warmup)

    if args.only == "csr":
        ms_csr, ms_one, ms_dense, dense_bytes, csr_bytes = bench_csr_conversion(
            capi, synth, args.steps, args.warmup)
        result["csr"] = {"dense_to_csr_two_calls_ms": ms_csr, "dense_to_csr_one_call_ms": ms_one,
                         "csr_to_dense_ms": ms_dense, "dense_bytes": dense_bytes,
                         "csr_bytes": csr_bytes}

    if args.only == "spgemm":
        ms, products, nnz_c, nbytes, nnz_a, nnz_b, one_ms = bench_spgemm(capi, synth, args.steps,
                                                                         args.warmup)
        result["spgemm"] = {"count_plus_fill_ms": ms, "one_call_ms": one_ms, "products": products,
                            "nnz_a": nnz_a,
                            "nnz_b": nnz_b, "nnz_c": nnz_c, "algorithmic_bytes": nbytes}

    if args.only in (None, "spmm"):
        sp_steps = max(args.steps * 4, 100)
        sp_event, sp_wall, d5, nnz, alg_bytes = bench_spmm(capi, synth, sp_steps, args.warmup)
        gbs = alg_bytes / (sp_event * 1e-3) / 1e9
        spmm = {
            "workload": "configuration 5: CSR 8192x8192 at 1 %% (nnz %d) x dense 8192x256 f32, "
                        "store mode" % nnz,
            "entry_point": "sph_spmm_csr_f32", "steps": sp_steps, "launch_ms": sp_event,
            "value": gbs, "unit": "GB/s", "gflops": 2.0 * nnz * 256 / (sp_event * 1e-3) / 1e9,
            "roofline": {"bound": "hbm", "kernel": "SpmmSlabVec4<16>", "achieved": gbs,
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                         "traffic": recorded_traffic("spmm_slab_config5.txt"),
                         "traffic_unit": "bytes per launch (profiles/spmm_slab_config5.txt)",
                         "algorithmic_bytes_per_launch": alg_bytes,
                         "gather_bytes_per_launch": nnz * 256 * 4,
                         "gather_path": spmm_gather_path(nnz, 256, sp_event, info)},
        }
        if not args.no_cpu and args.only is None:
            dt = cpu_spmm_baseline(d5)
            spmm["cpu_baseline"] = {"value": alg_bytes / dt / 1e9, "unit": "GB/s", "cores": 1,
                                    "kind": "port",
                                    "sample": "whole configuration 5, storage-order CSR loop "
                                              "(the reference has no sparse x dense code), %.2f s" % dt}
        result["spmm"] = spmm

    if args.only is None:
        # configurations 1, 2 and 4, each against the fp32 MFMA peak (configuration 1 is a
        # single 33.6 MFLOP launch and is bound by launch latency, not by any roofline)
        configs = {}
        c1 = synth.config1()
        ms = bench_f32(capi, c1["A"], c1["B"], c1["C"], 256, 256, 256, 1, 256 * 256, 1000, 50)
        configs["config1_f32_256"] = f32_roofline(
            "configuration 1: out[256,256] += A[256,256] * B[256,256] fp32, one launch",
            "sph_gemm_f32", "GemmF32SkinnyKernel", ms, 2.0 * 256 ** 3, 4 * 4 * 256 * 256)
        c2 = synth.config2()
        ms = bench_f32(capi, c2["A"], c2["B"], c2["C"], 512, 512, 512, 16, 0, 200, 20)
        configs["config2_f32_batched"] = f32_roofline(
            "configuration 2: out[16,512,512] += A[16,512,512] * B[1,512,512] fp32, B shared "
            "(stride 0), one launch", "sph_gemm_f32", "GemmF32DmaKernel<64>", ms,
            16 * 2.0 * 512 ** 3, 4 * 512 * 512 * (16 + 1 + 16 + 16))
        c4 = synth.config4()
        sizes = [c4["x"].shape[1]] + [w.shape[1] for w in c4["W"]]
        batch = c4["x"].shape[0]
        # x, W, bias read once, every layer's y written once and read once by the next layer
        mlp_bytes = 4 * (batch * sizes[0] + sum(sizes[l] * sizes[l + 1] + sizes[l + 1]
                                                for l in range(3))
                         + batch * (2 * sizes[1] + 2 * sizes[2] + sizes[3]))
        ms, fl = bench_mlp(capi, synth, 100, 10, fused=True)
        configs["config4_mlp_forward"] = f32_roofline(
            "configuration 4: 3-layer MLP forward 784-1024-1024-10 on x[1024,784] fp32, bias and "
            "ReLU fused into each layer's launch (3 launches per step)",
            "sph_linear_forward_f32 x 3", "GemmF32DmaKernel / GemmF32SkinnyKernel (fused epilogue)",
            ms, fl, mlp_bytes)
        ms, fl = bench_mlp(capi, synth, 100, 10)
        configs["config4_mlp_forward"]["reference_call_sequence"] = {
            "note": "the reference's operator calls one for one: fill, K = 1 bias GEMM, GEMM, "
                    "ReLU (11 launches per step); same result bits as the fused form",
            "launch_ms": ms, "tflops": fl / (ms * 1e-3) / 1e12}
        result["configs"] = configs

    if args.all and args.only is None:
        others = {}
        ms_ref, fl = bench_mlp_backward(capi, synth, 100, 10, direct=False)
        ms_dir, _ = bench_mlp_backward(capi, synth, 100, 10, direct=True)
        ms_fused, _ = bench_mlp_backward(capi, synth, 100, 10, direct=True, fused_update=True)
        others["config4_mlp_backward_sgd"] = {
            "reference_sequence_ms": ms_ref, "direct_ms": ms_dir,
            "direct_tflops": fl / (ms_dir * 1e-3) / 1e12,
            "direct_update_in_gemm_ms": ms_fused,
            "direct_update_in_gemm_tflops": fl / (ms_fused * 1e-3) / 1e12,
            "note": "reference sequence: Transpose + Gemm, Zeros, Scale + Sub; direct: "
                    "transposed-read / overwrite GEMM flags and the one-pass SGD step; "
                    "update in gemm: the weight and bias gradient products end in the SGD "
                    "step (sph_gemm_f32_sgd), no gradient is stored (bit-identical results "
                    "in all three)"}
        ms_f, _ = bench_mlp(capi, synth, 100, 10, fused=True, graph=True)
        ms_b, _ = bench_mlp_backward(capi, synth, 100, 10, direct=True, graph=True)
        others["config4_replayed_as_graphs"] = {
            "forward_fused_ms": ms_f, "backward_sgd_direct_ms": ms_b,
            "note": "the same call sequences recorded once with sph_graph_begin_capture / "
                    "sph_graph_end_capture and replayed with sph_graph_launch"}
        ms, nbytes = bench_sgd_step(capi, 200, 20)
        others["sgd_step_64MiB"] = {"launch_ms": ms, "gbs": nbytes / (ms * 1e-3) / 1e9,
                                    "frac_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS}
        ms_csr, ms_one, ms_dense, dense_bytes, csr_bytes = bench_csr_conversion(capi, synth, 50, 5)
        others["csr_conversion_config5"] = {
            "dense_to_csr_ms": ms_one,
            "dense_to_csr_gbs": (dense_bytes + csr_bytes) / (ms_one * 1e-3) / 1e9,
            "dense_to_csr_note": "sph_csr_from_dense_f32, one pass over the dense matrix; "
                                 "algorithmic bytes: dense read once + CSR written",
            "dense_to_csr_two_calls_ms": ms_csr,
            "dense_to_csr_two_calls_note": "sph_csr_row_offsets_f32 + sph_csr_fill_f32 read the "
                                           "dense matrix twice (count, then fill)",
            "csr_to_dense_ms": ms_dense,
            "csr_to_dense_gbs": (dense_bytes + csr_bytes) / (ms_dense * 1e-3) / 1e9}
        ms, products, nnz_c, nbytes, nnz_a, nnz_b, one_ms = bench_spgemm(capi, synth, 50, 5)
        others["spgemm_8192_8_per_row"] = {
            "one_call_ms": one_ms,
            "workload": "CSR 8192x8192 (nnz %d) x CSR 8192x8192 (nnz %d) -> CSR (nnz %d)"
                        % (nnz_a, nnz_b, nnz_c),
            "count_plus_fill_ms": ms, "products": products,
            "gproducts_per_s": 2 * products / (ms * 1e-3) / 1e9,
            "algorithmic_gbs": nbytes / (ms * 1e-3) / 1e9,
            "note": "both passes compute every product (the count pass must see which sums "
                    "cancel); products counted once per pass in gproducts_per_s"}
        ms, products, nnz_c, nbytes, nnz_a, nnz_b, one_ms = bench_spgemm(capi, synth, 20, 3, n=65536)
        others["spgemm_65536_8_per_row"] = {
            "one_call_ms": one_ms,
            "workload": "CSR 65536x65536 (nnz %d) x CSR 65536x65536 (nnz %d) -> CSR (nnz %d)"
                        % (nnz_a, nnz_b, nnz_c),
            "count_plus_fill_ms": ms, "products": products,
            "gproducts_per_s": 2 * products / (ms * 1e-3) / 1e9,
            "algorithmic_gbs": nbytes / (ms * 1e-3) / 1e9,
            "note": "16 strips wide: rows with few products go through the hash-table kernel"}
        ms, ms_product, nnz_w, ms_unfused = bench_sparse_linear(capi, synth, 50, 5)
        others["sparse_linear_forward_8192x8192_batch256"] = {
            "forward_ms": ms, "csr_x_dense_ms": ms_product, "launches_per_forward": 3,
            "weights_kept": nnz_w,
            "gflops": 2.0 * nnz_w * 256 / (ms * 1e-3) / 1e9,
            "note": "the NN::SparseLinearForward sequence through the C ABI: transpose x, CSR x "
                    "dense with the bias of an output row as the value the product is added to "
                    "(sph_spmm_csr_bias_f32), transpose y",
            "six_launch_form_ms": ms_unfused,
            "six_launch_form_note": "transpose x, ones, zero fill, bias x ones (K = 1 GEMM), CSR "
                                    "x dense (accumulating), transpose y: same result bits"}
        others["one_pass_kernels_4096x4096"] = bench_elementwise(capi, 50, 5)
        others["device_block_64MiB"] = bench_allocation(capi)
        result["others"] = others

    if not args.no_cpu and args.only is None:
        result["cpu_baseline"] = cpu_gemm_baseline(d3)
        result["cpu_baseline_all_cores"] = cpu_gemm_all_cores(d3)

    print(json.dumps(result))


if __name__ == "__main__":
    main()

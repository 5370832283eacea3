#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one pass of the A16W4 Llama-2-7B MLP block at 4 x 512 = 2048 bf16 tokens:
forward  down(silu(gate(x)) * up(x))  and the dX backward through all three projections
(six dequant-GEMM products, 1108.1 GFLOP, in the four launches the fused training block makes:
the bf16 glue of autograd sits in the GEMM epilogues), with synthetic seeded weights and
activations already resident in HBM. The headline value is GEMM TFLOP/s of that step. The same JSON line also
carries the kernel roofline of the dominant kernel (measured with HIP events on the launch
stream), HBM GB/s of the requantizer and of the decode GEMV sweep, the A8W8 GEMM rate, and
the CPU baseline (the torch restatement of the reference's dequant path on the host cores).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16 = 2.5e15   # dense bf16 MFMA, flop/s
PEAK_I8 = 5.0e15     # dense int8 MFMA, op/s
PEAK_HBM = 8.0e12    # byte/s

TOKENS, HID, FFN = 2048, 4096, 11008
GROUP = 128


def synth_w4(N, K, seed, device):
    g = torch.Generator(device="cpu").manual_seed(seed)
    codes = torch.randint(0, 256, (N * K // 2,), generator=g, dtype=torch.uint8).view(torch.int8)
    scales = (torch.randn(N * K // GROUP, 1, generator=g) * 0.02).abs().div(7).to(torch.bfloat16)
    scales = torch.where(scales == 0, torch.full_like(scales, 2.0 ** -10), scales)
    zeros = torch.randint(6, 10, (N * K // GROUP, 1), generator=g).to(torch.bfloat16)
    return codes.to(device), scales.to(device), zeros.to(device)


def event_time(fn, iters, warm=30, warm_seconds=0.08):
    """Average seconds per call of fn(), HIP events on the current (= launch) stream. The warm-up
    runs at least `warm` calls and at least `warm_seconds` of work: after an idle period the
    device takes tens of milliseconds to settle at its sustained clock (a GEMM timed over the
    first 5 ms reads ~10 % low)."""
    t0 = time.perf_counter()
    done = 0
    while done < warm or time.perf_counter() - t0 < warm_seconds:
        for _ in range(10):
            fn()
        done += 10
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / iters


def graph_time(calls, replays=20, warm_seconds=0.08):
    """Average seconds per kernel for launch-latency-scale kernels: the calls (one per rotating
    buffer set) are captured into one HIP graph so that launches are back to back, and the
    graph is replayed between two HIP events on the replay stream. The graph is first replayed for
    at least `warm_seconds` (the same settling time event_time gives its kernels: the inputs of these
    blocks are built on the host for seconds, with the device idle and its clock down), and the
    timed replays follow without a pause."""
    for c in calls:
        c()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for c in calls:
            c()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < warm_seconds:
        for _ in range(10):
            g.replay()
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(3):
        g.replay()
    e0.record()
    for _ in range(replays):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / (replays * len(calls))


class MLPBlock:
    """A16W4 Llama-2-7B MLP (gate/up 11008x4096, down 4096x11008) on the HIP kernels."""

    def __init__(self, device):
        from latentq_llm_amd import ops
        self.ops = ops
        self.gate = synth_w4(FFN, HID, 1, device)
        self.up = synth_w4(FFN, HID, 2, device)
        self.down = synth_w4(HID, FFN, 3, device)
        g = torch.Generator(device="cpu").manual_seed(4)
        self.x = torch.randn(TOKENS, HID, generator=g).to(torch.bfloat16).to(device)
        self.dy = torch.randn(TOKENS, HID, generator=g).to(torch.bfloat16).to(device)

    def step(self):
        """The block as latentq_llm_amd.fused_mlp.QuantLlamaMLP runs it in training: four launches, the bf16 glue
        of autograd (silu, three products, silu backward) in the GEMM epilogues and the sum of the two input
        gradients in one reduction over both products."""
        o = self.ops
        h, g, u = o.a16w4_gate_up_silu(self.x, self.gate, self.up, (FFN, HID), save=True)
        y = o.a16w4_forward(h, *self.down, (HID, FFN))
        dg, du = o.a16w4_dx_silu_bwd(self.dy, *self.down, (HID, FFN), g, u)
        dx = o.a16w4_dx_pair(dg, self.gate, du, self.up, (FFN, HID))
        return y, dx

    def step_events(self):
        """step() with a HIP event recorded on the launch stream before, between and after its four launches:
        returns the five events (the launches run back to back as in step(); an event is a timestamp packet)."""
        o = self.ops
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(5)]
        ev[0].record()
        h, g, u = o.a16w4_gate_up_silu(self.x, self.gate, self.up, (FFN, HID), save=True)
        ev[1].record()
        o.a16w4_forward(h, *self.down, (HID, FFN))
        ev[2].record()
        dg, du = o.a16w4_dx_silu_bwd(self.dy, *self.down, (HID, FFN), g, u)
        ev[3].record()
        o.a16w4_dx_pair(dg, self.gate, du, self.up, (FFN, HID))
        ev[4].record()
        return ev

    def step_unfused(self):
        """The same block layer by layer, with the bf16 glue exactly as autograd runs it (six GEMM launches and
        six tensor-library kernels)."""
        o = self.ops
        g = o.a16w4_forward(self.x, *self.gate, (FFN, HID))
        u = o.a16w4_forward(self.x, *self.up, (FFN, HID))
        act = torch.nn.functional.silu(g)
        h = act * u
        y = o.a16w4_forward(h, *self.down, (HID, FFN))
        dh = o.a16w4_dx(self.dy, *self.down, (HID, FFN))
        du = dh * act
        dg = torch.ops.aten.silu_backward(dh * u, g)
        dx = o.a16w4_dx(dg, *self.gate, (FFN, HID))
        dx += o.a16w4_dx(du, *self.up, (FFN, HID))
        return y, dx


MLP_FLOP = 6 * 2 * TOKENS * HID * FFN  # 1 108.1 GFLOP

# HBM traffic per GEMM launch: read from profiles/gemm_a16w4_c2_counters.json, which is written together
# with profiles/gemm_a16w4_c2_counters.md from two counter runs of
#   rocprofv3 --pmc FETCH_SIZE -- python3 bench.py --profile-target gemm     (then WRITE_SIZE)
# each scaled by what the same counter reads for the 256 MiB calibration copy of the same run.
PMC_LAUNCHES = ("fwd_gate_up_silu", "fwd_down", "dx_down_silu_bwd", "dx_gate_up_pair")  # the four launches of a step


def gemm_traffic_bytes():
    """Mean HBM bytes (read + written) per product of the MLP step (its four launches hold six), or None when the
    counter summary is missing."""
    path = os.path.join(ROOT, "profiles", "gemm_a16w4_c2_counters.json")
    try:
        with open(path) as f:
            mb = json.load(f)["hbm_MB_per_launch"]
        tot = sum(mb[k]["read"] + mb[k]["written"] for k in PMC_LAUNCHES)
    except (OSError, KeyError, ValueError):
        return None
    return tot * 1e6 / 6


def _requant_sets(device, N, K, nb, seed0):
    sets = []
    for i in range(nb):
        p, s, z = synth_w4(N, K, seed0 + i, device)
        g = (torch.randn(N, K, device=device) * 1e-3).to(torch.bfloat16)
        sets.append((p, s, z, g, torch.empty_like(p)))
    return sets


def bench_requant(device):
    from latentq_llm_amd import _C, ops
    N, K = 8192, 2048
    nb = 8  # 8 x 50 MB of distinct buffers > 256 MB of last-level cache
    sets = _requant_sets(device, N, K, nb, 10)
    calls = [(lambda t=t, i=i: ops.requant_sr(t[0], t[1], t[2], t[3], 1e-4, (N, K), seed=7, offset=i, out=t[4]))
             for i, t in enumerate(sets)]
    sec = graph_time(calls)
    nbytes = N * K // 2 * 2 + N * K * 2 + 4 * N * K // GROUP
    # a plain copy that moves the same number of bytes (half read, half written), same rotation
    half = (nbytes // 2) // 16 * 16
    bufs = [(torch.empty(half, dtype=torch.uint8, device=device).random_(0, 256), torch.empty(half, dtype=torch.uint8, device=device))
            for _ in range(nb)]
    for src, dst in bufs:
        assert src.numel() == half and dst.numel() == half and src.data_ptr() % 16 == 0 and dst.data_ptr() % 16 == 0
    copies = [(lambda b=b: _C.call("lq_calib_copy", b[0].data_ptr(), b[1].data_ptr(), half,
                                   torch.cuda.current_stream().cuda_stream)) for b in bufs]
    sec_copy = graph_time(copies)
    del bufs
    return {"shape": [N, K], "us": sec * 1e6, "GB/s": nbytes / sec / 1e9, "frac_hbm": nbytes / sec / PEAK_HBM,
            "bytes": nbytes, "noise": "in-kernel Philox4x32-10, 16-bit draws",
            "copy_same_bytes_us": sec_copy * 1e6, "frac_of_copy": sec_copy / sec}


def bench_gradq8(device):
    """The 8-bit gradient accumulator on a dW of the MLP (11008 x 4096): set_value and add_ forms."""
    from latentq_llm_amd import ops
    N, K = FFN, HID
    sets = []
    for i in range(4):
        dw = (torch.randn(N, K, device=device) * 1e-3).to(torch.bfloat16)
        sets.append((dw, torch.empty((N, K), dtype=torch.int8, device=device),
                     torch.empty((N, 1), dtype=torch.bfloat16, device=device)))
    out = {"shape": [N, K]}
    for name, acc, nbytes in (("set", False, 3 * N * K), ("add", True, 4 * N * K)):
        for t in sets:
            ops.gradq8_quant(t[0], t[1], t[2], False, seed=1, offset=0)
        sec = graph_time([(lambda t=t, i=i: ops.gradq8_quant(t[0], t[1], t[2], acc, seed=1, offset=i)) for i, t in enumerate(sets)])
        out[name] = {"us": sec * 1e6, "GB/s": nbytes / sec / 1e9, "frac_hbm": nbytes / sec / PEAK_HBM, "bytes": nbytes}
    return out


def bench_latent(device):
    """The two fused passes of the exact 4-bit-residual latent mode (lbit = 4) on the requantizer's shape."""
    from latentq_llm_amd import ops
    N, K = 8192, 2048
    curve = (2, 0.125, 2, 0.25, 4)  # k1, b1, k2, b2, k3 of the default companding curve
    sets = []
    for i in range(8):
        p, s, z = synth_w4(N, K, 40 + i, device)
        res = torch.randint(-2 ** 31, 2 ** 31 - 1, (N * K // 8,), device=device, dtype=torch.int64).to(torch.int32)
        lat = ops.latent_w4_reconstruct(p, s, z, res, (N, K), *curve)
        sets.append((p, s, z, res, lat))
    nbytes = N * K // 2 + N * K // 2 + N * K * 2 + 4 * N * K // GROUP
    out = {"shape": [N, K], "bytes": nbytes}
    for name, calls in [
        ("reconstruct", [(lambda t=t: ops.latent_w4_reconstruct(t[0], t[1], t[2], t[3], (N, K), *curve)) for t in sets]),
        ("requant", [(lambda t=t: ops.latent_w4_requant(t[4], t[1], t[2], t[3], (N, K), *curve)) for t in sets]),
    ]:
        sec = graph_time(calls)
        out[name] = {"us": sec * 1e6, "GB/s": nbytes / sec / 1e9, "frac_hbm": nbytes / sec / PEAK_HBM}
    return out


def bench_gemv(device):
    """configs[4]: the decode GEMV over the three 7B matrix shapes at 1, 4 and 16 tokens, as HIP graphs over
    rotating weight sets larger than the last-level cache. Beside every point: a read-only launch over buffers
    of the same rotation holding the same number of bytes (lq_calib_read, one 16-byte load per thread: the
    GEMV's own access shape), i.e. what it costs on this device just to read what the kernel must read."""
    from latentq_llm_amd import _C, ops
    out = []
    sink = torch.zeros(64, dtype=torch.int32, device=device)
    for (N, K) in [(4096, 4096), (11008, 4096), (4096, 11008)]:
        nb = int(300e6 // (N * K // 2)) + 1
        ws = [synth_w4(N, K, 20 + i, device) for i in range(nb)]
        for M in (1, 4, 16):
            x = torch.randn(M, K, device=device).to(torch.bfloat16)
            ys = [torch.empty(M, N, device=device, dtype=torch.bfloat16) for _ in range(nb)]
            calls = [(lambda w=w, y=y: ops.a16w4_forward(x, *w, (N, K), out=y)) for w, y in zip(ws, ys)]
            sec = graph_time(calls)
            nbytes = N * K // 2 + 4 * N * K // GROUP + 2 * M * K + 2 * M * N
            rbytes = nbytes // 16 * 16
            bufs = [torch.empty(rbytes, dtype=torch.uint8, device=device).random_(0, 256) for _ in range(nb)]
            reads = [(lambda b=b: _C.call("lq_calib_read", b.data_ptr(), rbytes, 0, sink.data_ptr(),
                                          torch.cuda.current_stream().cuda_stream)) for b in bufs]
            sec_read = graph_time(reads)
            del bufs
            out.append({"N": N, "K": K, "M": M, "us": sec * 1e6, "GB/s": nbytes / sec / 1e9,
                        "frac_hbm": nbytes / sec / PEAK_HBM, "read_same_bytes_us": sec_read * 1e6,
                        "frac_of_read": sec_read / sec})
        del ws
    return out


def bench_a8w8(device):
    from latentq_llm_amd import ops
    M = TOKENS
    out = []
    for (N, K) in [(2048, 2048), (8192, 2048), (2048, 8192)]:
        # HIP graphs over rotating weight matrices, 0.4 GB of them (the weights come from HBM, as in any real use; the
        # activations are where the previous kernel left them), and over one matrix (everything cached) for comparison
        nb = (400 << 20) // (N * K) + 1
        sx = (torch.randn(M, device=device) * 0.05).abs()
        sw = (torch.randn(N, device=device) * 0.01).abs()
        x8 = torch.randint(-127, 128, (M, K), device=device, dtype=torch.int8)
        ws = [torch.randint(-127, 128, (N, K), device=device, dtype=torch.int8) for _ in range(nb)]
        sec = graph_time([(lambda w=w: ops.a8w8_forward(x8, w, sx, sw)) for w in ws])
        sec_cached = graph_time([(lambda: ops.a8w8_forward(x8, ws[0], sx, sw)) for _ in range(8)])
        del ws
        out.append({"M": M, "N": N, "K": K, "us": sec * 1e6, "TOP/s": 2 * M * N * K / sec / 1e12,
                    "frac_mfma_i8": 2 * M * N * K / sec / PEAK_I8, "weight_matrices": nb, "us_cached_weights": sec_cached * 1e6})
    # what the int8 matrix pipes deliver with nothing else in the loop (random and all-zero operands, two waves per SIMD)
    ceil = {}
    for name, zero in (("random_operands", False), ("zero_operands", True)):
        tops, ghz = mfma_loop_i8(device, zero)
        ceil[f"mfma_loop_i8_{name}"] = {"TOP/s": tops, "clock_GHz": ghz}
    loop = ceil["mfma_loop_i8_random_operands"]["TOP/s"]
    for rec in out:
        rec["achieved_over_ceiling"] = rec["TOP/s"] / loop
    out.append({"ceiling": ceil})
    # the activation quantisers in front of the GEMM (bf16 -> int8): given clamp value, the tensor's own maximum
    # found on the device (two launches), one scale per token row
    # (ten activation tensors in turn: 0.5 GB with their outputs, more than the last-level cache holds)
    xs = [torch.randn(M, 8192, device=device).to(torch.bfloat16) for _ in range(10)]
    numel = xs[0].numel()
    clampv = xs[0].float().abs().max().reshape(1)
    sec = event_time(_rotate([(lambda x=x: ops.act_quant_i8(x, clampv)) for x in xs]), 20)
    out.append({"act_quant": [M, 8192], "us": sec * 1e6, "GB/s": 3 * numel / sec / 1e9})
    sec = event_time(_rotate([(lambda x=x: ops.act_quant_i8_dynamic(x)) for x in xs]), 20)
    out.append({"act_quant_dynamic": [M, 8192], "us": sec * 1e6, "GB/s": 5 * numel / sec / 1e9,
                "bytes_per_element": 5, "what": "max pass (2 B read) + quantise pass (2 B read, 1 B written; the second read may come from the last-level cache)"})
    sec = event_time(_rotate([(lambda x=x: ops.act_quant_i8_per_token(x)) for x in xs]), 20)
    out.append({"act_quant_per_token": [M, 8192], "us": sec * 1e6, "GB/s": 3 * numel / sec / 1e9})
    x8s = [ops.act_quant_i8_per_token(x) for x in xs]
    sec = event_time(_rotate([(lambda t=t: ops.act_dequant_i8(t[0], t[1], True)) for t in x8s]), 20)
    out.append({"act_dequant": [M, 8192], "us": sec * 1e6, "GB/s": 3 * numel / sec / 1e9})
    s127 = (127. / clampv.to(torch.bfloat16)).reshape(1)
    sec = event_time(_rotate([(lambda x=x: ops.act_fake_quant(x, s127)) for x in xs]), 20)
    out.append({"act_fake_quant": [M, 8192], "us": sec * 1e6, "GB/s": 4 * numel / sec / 1e9})
    return out


def bench_a8w8_layer_step(device):
    """One A8W8 layer's training micro-step at the configs[3] shapes (not part of `value`): forward, input gradient and
    weight gradient accumulated in bf16, on the library's kernels and as the tensor-operation chain the reference's
    Functions run (utils/quant.py:254-293 with backward_hook_fn; the vendor's int8 product standing in for its
    external GEMM, and without the host synchronisation its `.item()` costs). Wall time of the launches from the
    host: for the smallest shape that is launch overhead as much as kernel time."""
    from latentq_llm_amd import ops
    M, out = TOKENS, []
    for (N, K) in [(2048, 2048), (8192, 2048), (2048, 8192)]:
        g = torch.Generator(device="cpu").manual_seed(N + K)
        x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(device)
        dy = torch.randn(M, N, generator=g).to(torch.bfloat16).to(device)
        w8 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).to(device)
        qs = (torch.rand(N, 1, generator=g) * 0.01 + 1e-3).to(torch.bfloat16).to(device)
        grad = torch.zeros(N, K, dtype=torch.bfloat16, device=device)

        def fused():
            x8, sx, work = ops.act_quant_i8_dynamic(x, True)
            ops.a8w8_forward(x8, w8, sx, qs.view(-1))
            xf = ops.act_dequant_i8(x8, work[1:2], False)
            ops.a8w8_dx(dy, w8, qs.view(-1))
            ops.weight_grad_acc(dy, xf, grad)

        def chain():
            clampv = x.max()
            x8 = (x * 127. / clampv).round_().clamp_(-128, 127).to(torch.int8)
            acc = torch._int_mm(x8, w8.t())
            _ = ((acc.float() * (clampv.float() / 127.)).to(torch.bfloat16)) * qs.view(1, -1)
            xf = x8.to(torch.bfloat16) * (clampv / 127.)
            wf = (w8.to(torch.bfloat16) * qs).to(torch.bfloat16)
            dy.mm(wf)
            grad.add_(dy.t().mm(xf))
        out.append({"N": N, "K": K, "library_kernels_us": event_time(fused, 20) * 1e6,
                    "tensor_op_chain_us": event_time(chain, 20) * 1e6})
    return out


def _rotate(calls):
    """A callable that runs the next of `calls` each time (operand sets larger than the last-level cache in turn)."""
    state = {"i": -1}

    def run():
        state["i"] = (state["i"] + 1) % len(calls)
        calls[state["i"]]()
    return run


def bench_adam8(device):
    """One Adam step on uint8 block-wise moments over 8192 x 2048 elements: the fused kernel and, for
    scale, the chain of tensor operations it replaces (latentq_llm_amd.quant with FUSED_ADAM8 off); then the whole
    optimizer step of an lbit = 4 layer as one kernel, for 4-bit and for 8-bit weights. Every launch works on the
    next of four operand sets (0.5-0.7 GB together: operands come from HBM, not from the last-level cache)."""
    from latentq_llm_amd import ops, quant as q
    N, K = 8192, 2048
    n, block = N * K, 2048
    nblk = n // block
    curve = (2, 0.1875, 3, 0.375, 3)
    sets = []
    for i in range(4):
        t = {"grad": (torch.randn(n, device=device) * 1e-3).to(torch.bfloat16),
             "param": (torch.randn(n, device=device) * 0.02).to(torch.bfloat16),
             "s1": torch.randint(0, 256, (n,), device=device, dtype=torch.uint8),
             "s2": torch.randint(0, 256, (n,), device=device, dtype=torch.uint8),
             "sc1": torch.full((nblk, 1), 1e-5, device=device), "mx1": torch.full((nblk, 1), 1.3e-3, device=device),
             "sc2": torch.full((nblk, 1), 1e-5, device=device), "mx2": torch.full((nblk, 1), 2.6e-3, device=device),
             "res": torch.randint(-2**31, 2**31 - 1, (n // 8,), device=device, dtype=torch.int64).to(torch.int32),
             "w8": torch.randint(-128, 128, (N, K), device=device, dtype=torch.int8),
             "qs": ((torch.randn(N, device=device) * 0.01).abs() + 1e-3).to(torch.bfloat16)}
        t["codes"], t["scales"], t["zeros"] = synth_w4(N, K, 7 + i, device)
        sets.append(t)
    mom = lambda t: (t["s1"], t["s2"], t["sc1"], t["mx1"], t["sc2"], t["mx2"])
    sec = event_time(_rotate([(lambda t=t: ops.adam8_update(t["grad"], *mom(t), 0.9, 0.95, 1e-8, 1e-3, param=t["param"]))
                              for t in sets]), 20)
    nbytes = 10 * n + 32 * nblk

    def chain(t=sets[0]):
        m = q.DeQfunc_8bit_opt(t["s1"], [t["sc1"], t["mx1"]]).to(torch.bfloat16)
        v = q.DeQfunc_8bit_opt(t["s2"], [t["sc2"], t["mx2"]])
        v = (v * v).to(torch.bfloat16)
        m.mul_(0.9).add_(t["grad"], alpha=0.1)
        v.mul_(0.95).addcmul_(t["grad"], t["grad"], value=0.05)
        d = v.sqrt_().add_(1e-8)
        t["param"].addcdiv_(m, d, value=-1e-3)
        q.Qfunc_8bit_opt(m.float(), blocksize=nblk)
        q.Qfunc_8bit_opt(d.float(), blocksize=nblk)
    sec_chain = event_time(chain, 5, warm=2)
    # the whole optimizer step of an lbit = 4 layer as one kernel: codes + residual words in and out.
    # per element: 2 B of gradient, 2 + 2 B of moments in and out, 0.5 + 0.5 B of codes and of residual in and out
    sec_step = event_time(_rotate([(lambda t=t: ops.adam8_latent_w4_step(
        t["grad"], t["codes"], t["res"], t["scales"].view(-1), t["zeros"].view(-1), (N, K), *mom(t), curve, curve,
        0.9, 0.95, 1e-8, 1e-3)) for t in sets]), 20)
    step_bytes = 8 * n + 32 * nblk + 4 * n // 128
    # the same for an 8-bit-weight layer (int8 codes, one scale per row): the single kernel against its three passes
    sec_w8 = event_time(_rotate([(lambda t=t: ops.adam8_latent_w8_step(
        t["grad"], t["w8"], t["res"], t["qs"], *mom(t), curve, curve, 0.9, 0.95, 1e-8, 1e-3)) for t in sets]), 20)

    def three_passes(t):
        lat = ops.latent_w8_reconstruct(t["w8"], t["qs"], t["res"], *curve)
        ops.adam8_update(t["grad"], *mom(t), 0.9, 0.95, 1e-8, 1e-3, param=lat.view(-1))
        ops.latent_w8_requant(lat, t["qs"], t["res"], *curve)
    sec_w8_3 = event_time(_rotate([(lambda t=t: three_passes(t)) for t in sets]), 20)
    w8_bytes = 9 * n + 32 * nblk + 2 * N  # as above with 1 + 1 B of codes
    return {"elements": n, "block": block, "bytes": nbytes, "us": sec * 1e6, "GB/s": nbytes / sec / 1e9,
            "frac_hbm": nbytes / sec / PEAK_HBM, "tensor_op_chain_us": sec_chain * 1e6, "operand_sets": len(sets),
            "latent_w4_step": {"bytes": step_bytes, "us": sec_step * 1e6, "GB/s": step_bytes / sec_step / 1e9,
                               "frac_hbm": step_bytes / sec_step / PEAK_HBM},
            "latent_w8_step": {"bytes": w8_bytes, "us": sec_w8 * 1e6, "GB/s": w8_bytes / sec_w8 / 1e9,
                               "frac_hbm": w8_bytes / sec_w8 / PEAK_HBM, "three_passes_us": sec_w8_3 * 1e6}}


def bench_dw(device):
    """dW = dY^T X of the two MLP shapes (not part of `value`): the library's own GEMM (operands read as they lie),
    the same with the int8 accumulator's add_ or the bf16 gradient's add_ as its epilogue, and for scale the vendor GEMM on the strided view (as
    the reference calls it) and on a transposed copy of dY."""
    from latentq_llm_amd import ops
    out = []
    for (N, K) in [(FFN, HID), (HID, FFN)]:
        # five operand / output sets in turn (0.9 GB: dY, X and the gradient come from HBM, as inside a training step)
        sets = [(torch.randn(TOKENS, N, device=device).to(torch.bfloat16), torch.randn(TOKENS, K, device=device).to(torch.bfloat16),
                 torch.zeros((N, K), dtype=torch.bfloat16, device=device), torch.zeros((N, K), dtype=torch.int8, device=device))
                for _ in range(5)]
        dy, x = sets[0][0], sets[0][1]
        flop = 2 * TOKENS * N * K
        t_ref = event_time(_rotate([(lambda t=t: t[0].t().mm(t[1])) for t in sets]), 20)
        t_tr = event_time(_rotate([(lambda t=t: ops.transpose_bf16(t[0]).mm(t[1])) for t in sets]), 20)
        t_new = event_time(_rotate([(lambda t=t: ops.weight_grad(t[0], t[1])) for t in sets]), 20)
        t_cached = event_time(lambda: ops.weight_grad(dy, x), 20)
        sc = torch.full((N, 1), 1e-3, dtype=torch.bfloat16, device=device)
        t_acc = event_time(_rotate([(lambda t=t: ops.weight_grad_acc8(t[0], t[1], t[3], sc, seed=1, offset=0)) for t in sets]), 20)
        t_add = event_time(_rotate([(lambda t=t: ops.weight_grad_acc(t[0], t[1], t[2])) for t in sets]), 20)  # grad.add_(dW) as the epilogue
        t_add_sep = event_time(_rotate([(lambda t=t: t[2].add_(ops.weight_grad(t[0], t[1]))) for t in sets]), 20)  # product stored, then added
        del sets
        out.append({"N": N, "K": K, "strided_mm_us": t_ref * 1e6, "strided_mm_TFLOP/s": flop / t_ref / 1e12,
                    "transposed_copy_mm_us": t_tr * 1e6, "transposed_copy_mm_TFLOP/s": flop / t_tr / 1e12,
                    "weight_grad_us": t_new * 1e6, "weight_grad_TFLOP/s": flop / t_new / 1e12,
                    "frac_mfma_bf16": flop / t_new / PEAK_BF16, "weight_grad_cached_operands_us": t_cached * 1e6,
                    "weight_grad_acc8_us": t_acc * 1e6, "weight_grad_acc8_TFLOP/s": flop / t_acc / 1e12,
                    "weight_grad_acc_bf16_us": t_add * 1e6, "weight_grad_then_add_us": t_add_sep * 1e6})
    return out


def _clock_ghz(clocks, n):
    """Median over n records (cycles start, cycles end, 100 MHz ticks start, ticks end) of the shader clock."""
    c = clocks[: 4 * n].view(n, 4).double()
    ticks = (c[:, 3] - c[:, 2]).clamp_min(1)
    return float(((c[:, 1] - c[:, 0]) / ticks * 0.1).median())


def mfma_loop(device, zero_operands, wgs_per_cu=2, seconds=0.004):
    """The MFMA-only loop (lq_calib_mfma_loop) under sustained load: (TFLOP/s, granted shader clock in GHz)."""
    import ctypes
    from latentq_llm_amd import _C
    n = 1 << 20
    if zero_operands:
        a = torch.zeros(n, dtype=torch.bfloat16, device=device)
        b = torch.zeros(n, dtype=torch.bfloat16, device=device)
    else:
        a = torch.randn(n, device=device).to(torch.bfloat16)
        b = (torch.randn(n, device=device) * 0.02).to(torch.bfloat16)
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    waves = 4 * cus * wgs_per_cu
    clocks = torch.zeros(4 * waves, dtype=torch.int64, device=device)
    sink = torch.zeros(waves, dtype=torch.float32, device=device)
    nw = ctypes.c_int64()
    st = torch.cuda.current_stream().cuda_stream

    def run(iters):
        _C.call("lq_calib_mfma_loop", a.data_ptr(), b.data_ptr(), n, iters, wgs_per_cu, clocks.data_ptr(), clocks.numel(),
                sink.data_ptr(), ctypes.addressof(nw), st)
    iters = 20000
    sec = event_time(lambda: run(iters), 5, warm=3, warm_seconds=0.1)
    flop = waves * iters * 8 * 32768.0
    return flop / sec / 1e12, _clock_ghz(clocks, waves)


def mfma_loop_i8(device, zero_operands, wgs_per_cu=2):
    """The MFMA-only loop on the int8 instruction (lq_calib_mfma_loop_i8): (TOP/s, granted shader clock in GHz)."""
    import ctypes
    from latentq_llm_amd import _C
    n = 1 << 20
    if zero_operands:
        a = torch.zeros(n, dtype=torch.int8, device=device)
        b = torch.zeros(n, dtype=torch.int8, device=device)
    else:
        a = torch.randint(-127, 128, (n,), dtype=torch.int8, device=device)
        b = torch.randint(-127, 128, (n,), dtype=torch.int8, device=device)
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    waves = 4 * cus * wgs_per_cu
    clocks = torch.zeros(4 * waves, dtype=torch.int64, device=device)
    sink = torch.zeros(waves, dtype=torch.int32, device=device)
    nw = ctypes.c_int64()
    st = torch.cuda.current_stream().cuda_stream
    iters = 20000
    sec = event_time(lambda: _C.call("lq_calib_mfma_loop_i8", a.data_ptr(), b.data_ptr(), n, iters, wgs_per_cu, clocks.data_ptr(),
                                     clocks.numel(), sink.data_ptr(), ctypes.addressof(nw), st), 5, warm=3, warm_seconds=0.1)
    ops_total = waves * iters * 8 * 65536.0
    return ops_total / sec / 1e12, _clock_ghz(clocks, waves)


def gemm_clock(device, backward, a, w, shape):
    """Shader clock granted to the dequant-GEMM under sustained load: 40 plain launches, then one that records
    each workgroup's cycle and real-time counters."""
    import ctypes
    from latentq_llm_amd import _C, ops
    N, K = shape
    M = a.shape[0]
    out = torch.empty((M, K if backward else N), dtype=torch.bfloat16, device=device)
    fn = (lambda: ops.a16w4_dx(a, *w, shape, out=out)) if backward else (lambda: ops.a16w4_forward(a, *w, shape, out=out))
    event_time(fn, 10)
    clocks = torch.zeros(4 * 4096, dtype=torch.int64, device=device)
    nwg = ctypes.c_int64()
    for _ in range(40):
        fn()
    _C.call("lq_calib_gemm_clocks", int(backward), a.data_ptr(), w[0].data_ptr(), w[1].data_ptr(), w[2].data_ptr(),
            out.data_ptr(), M, N, K, GROUP, clocks.data_ptr(), clocks.numel(), ctypes.addressof(nwg),
            torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return _clock_ghz(clocks, nwg.value)


def bench_ceiling(device, blk, h):
    """What the matrix pipes deliver with nothing else in the loop, at the clock the chip grants for it, next
    to the clock it grants the two dequant-GEMM kernels and to the vendor's dense bf16 GEMM on the same shapes."""
    out = {}
    for name, zero in (("random_operands", False), ("zero_operands", True)):
        for wgs in (2, 1):
            tf, ghz = mfma_loop(device, zero, wgs)
            out[f"mfma_loop_{name}_{wgs}wg_per_cu"] = {"TFLOP/s": tf, "clock_GHz": ghz}
    out["clock_GHz"] = {
        "fwd_gate_up": gemm_clock(device, False, blk.x, blk.gate, (FFN, HID)),
        "fwd_down": gemm_clock(device, False, h, blk.down, (HID, FFN)),
        "dx_gate_up": gemm_clock(device, True, h, blk.gate, (FFN, HID)),
        "dx_down": gemm_clock(device, True, blk.dy, blk.down, (HID, FFN)),
    }
    # vendor dense bf16 GEMM (torch.mm -> hipBLASLt) on the four shapes, weights N(0, 0.02^2), no dequantisation
    wg = (torch.randn(FFN, HID, device=device) * 0.02).to(torch.bfloat16)
    wd = (torch.randn(HID, FFN, device=device) * 0.02).to(torch.bfloat16)
    flop = 2 * TOKENS * HID * FFN
    vend = {}
    for name, fn in (("fwd_gate_up", lambda: blk.x.mm(wg.t())), ("fwd_down", lambda: h.mm(wd.t())),
                     ("dx_gate_up", lambda: h.mm(wg)), ("dx_down", lambda: blk.dy.mm(wd))):
        sec = event_time(fn, 30)
        vend[name] = {"us": sec * 1e6, "TFLOP/s": flop / sec / 1e12}
    out["vendor_dense_bf16_mm"] = vend
    return out


def bench_gate_up(device, blk):
    """silu(gate(x)) * up(x) of the 7B MLP as one launch (lq_a16w4_gate_up_silu, the inference-side fused product)
    against the same result from two forward GEMMs and torch's bf16 silu and product, over the token count."""
    from latentq_llm_amd import ops
    out = []
    for M in (256, 512, 1024, 2048, 4096):
        g = torch.Generator(device="cpu").manual_seed(40 + M)
        x = torch.randn(M, HID, generator=g).to(torch.bfloat16).to(device)
        h = torch.empty((M, FFN), dtype=torch.bfloat16, device=device)
        t_fused = event_time(lambda: ops.a16w4_gate_up_silu(x, blk.gate, blk.up, (FFN, HID), out=h), 30)
        t_parts = event_time(lambda: torch.nn.functional.silu(ops.a16w4_forward(x, *blk.gate, (FFN, HID)))
                             * ops.a16w4_forward(x, *blk.up, (FFN, HID)), 30)
        flop = 4.0 * M * HID * FFN
        out.append({"M": M, "fused_us": t_fused * 1e6, "fused_TFLOP/s": flop / t_fused / 1e12,
                    "two_gemms_silu_mul_us": t_parts * 1e6, "two_gemms_silu_mul_TFLOP/s": flop / t_parts / 1e12})
    # decode: one GEMV pass over both matrices against two GEMVs and the two tensor operations, as HIP graphs over
    # rotating weight sets larger than the last-level cache
    sets = [(synth_w4(FFN, HID, 70 + 2 * i, device), synth_w4(FFN, HID, 71 + 2 * i, device)) for i in range(7)]
    for M in (1, 4, 16):
        x = torch.randn(M, HID, device=device).to(torch.bfloat16)
        h = torch.empty((M, FFN), dtype=torch.bfloat16, device=device)
        g_, u_ = torch.empty_like(h), torch.empty_like(h)
        t_fused = graph_time([(lambda w=w: ops.a16w4_gate_up_silu(x, w[0], w[1], (FFN, HID), out=h)) for w in sets])

        def parts(w):
            ops.a16w4_forward(x, *w[0], (FFN, HID), out=g_)
            ops.a16w4_forward(x, *w[1], (FFN, HID), out=u_)
            torch.mul(torch.nn.functional.silu(g_), u_, out=h)
        t_parts = graph_time([(lambda w=w: parts(w)) for w in sets])
        nbytes = 2 * (FFN * HID // 2 + 4 * FFN * HID // GROUP) + 2 * M * HID + 2 * M * FFN
        out.append({"M": M, "fused_us": t_fused * 1e6, "fused_GB/s": nbytes / t_fused / 1e9, "fused_frac_hbm": nbytes / t_fused / 8e12,
                    "two_gemvs_silu_mul_us": t_parts * 1e6, "bytes": nbytes})
    return out


def bench_c0(device):
    """configs[0] (the reference's own CPU-runnable case: 3072 x 768 at 1024 tokens) on the GPU: forward and dX."""
    from latentq_llm_amd import ops
    N0, K0, M0 = 3072, 768, 1024
    w = synth_w4(N0, K0, 5, device)
    x = torch.randn(M0, K0, device=device).to(torch.bfloat16)
    dy = torch.randn(M0, N0, device=device).to(torch.bfloat16)
    tf = graph_time([lambda: ops.a16w4_forward(x, *w, (N0, K0))] * 8)
    td = graph_time([lambda: ops.a16w4_dx(dy, *w, (N0, K0))] * 8)
    flop = 2.0 * M0 * N0 * K0
    return {"workload": "configs[0]: 3072x768 at 1024 tokens", "fwd_us": tf * 1e6, "dx_us": td * 1e6,
            "TFLOP/s": 2 * flop / (tf + td) / 1e12, "plans": [ops.a16w4_plan(M0, (N0, K0))[0], ops.a16w4_plan(M0, (N0, K0), backward=True)[0]]}


def bench_copy(device):
    """Plain streaming copy (lq_calib_copy) over buffers larger than the last-level cache: the
    HBM rate this device sustains for read + write traffic, for comparison with the 8 TB/s peak."""
    from latentq_llm_amd import _C
    nbytes = 1 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device=device).random_(0, 256)
    dst = torch.empty_like(src)
    st = torch.cuda.current_stream().cuda_stream
    sec = event_time(lambda: _C.call("lq_calib_copy", src.data_ptr(), dst.data_ptr(), nbytes, st), 10, warm=3)
    return {"bytes_each_way": nbytes, "us": sec * 1e6, "GB/s": 2 * nbytes / sec / 1e9}


def profile_target(device, which, launches=10):
    """A short, fixed sequence of launches for a profiler run (kernel trace or counters): the
    calibration copy first, then the kernels of the named family, `launches` times each."""
    from latentq_llm_amd import _C, ops as o
    st = torch.cuda.current_stream().cuda_stream
    nbytes = 256 << 20
    src = torch.empty(nbytes, dtype=torch.uint8, device=device).random_(0, 256)
    dst = torch.empty_like(src)
    for _ in range(launches):
        _C.call("lq_calib_copy", src.data_ptr(), dst.data_ptr(), nbytes, st)
    del src, dst
    if which == "gemm":
        # every launch of the benchmark step, and the plain-store forms of the same products, 10 times each in this order
        # (launches that share a kernel name and grid are told apart by their position in the sequence)
        blk = MLPBlock(device)
        h = torch.randn(TOKENS, FFN, device=device).to(torch.bfloat16)
        for _ in range(launches):
            o.a16w4_forward(blk.x, *blk.gate, (FFN, HID))                      # 1 forward gate (or up), plain
        for _ in range(launches):
            o.a16w4_forward(h, *blk.down, (HID, FFN))                          # 2 forward down
        for _ in range(launches):
            o.a16w4_dx(h, *blk.gate, (FFN, HID))                               # 3 dX gate, plain store
        for _ in range(launches):
            o.a16w4_dx(blk.dy, *blk.down, (HID, FFN))                          # 4 dX down, plain store
        hbuf = torch.empty((TOKENS, FFN), dtype=torch.bfloat16, device=device)
        for _ in range(launches):
            _, g_, u_ = o.a16w4_gate_up_silu(blk.x, blk.gate, blk.up, (FFN, HID), out=hbuf, save=True)  # 5 fused gate / up, stores g, u, h
        for _ in range(launches):
            dg_, du_ = o.a16w4_dx_silu_bwd(blk.dy, *blk.down, (HID, FFN), g_, u_)  # 6 dX down with the silu-backward epilogue
        dxb = torch.zeros((TOKENS, HID), dtype=torch.bfloat16, device=device)
        for _ in range(launches):
            o.a16w4_dx(du_, *blk.up, (FFN, HID), out=dxb, accumulate=True)     # 7 dX up, accumulating
        for _ in range(launches):
            o.a16w4_dx_pair(dg_, blk.gate, du_, blk.up, (FFN, HID), out=dxb)   # 8 dX of gate and up in one reduction
        x1536 = torch.randn(1536, HID, device=device).to(torch.bfloat16)
        for _ in range(launches):
            o.a16w4_forward(x1536, *blk.gate, (FFN, HID))                      # 9 forward gate at 1536 tokens (128 x 128 tiles)
    elif which == "dw":
        # the weight-gradient GEMM on the two MLP shapes: plain store, then the int8 accumulate epilogue
        for (N, K) in [(FFN, HID), (HID, FFN)]:
            dy = torch.randn(TOKENS, N, device=device).to(torch.bfloat16)
            x = torch.randn(TOKENS, K, device=device).to(torch.bfloat16)
            q8 = torch.zeros((N, K), dtype=torch.int8, device=device)
            sc = torch.full((N, 1), 1e-3, dtype=torch.bfloat16, device=device)
            for _ in range(launches):
                o.weight_grad(dy, x)
            for i in range(launches):
                o.weight_grad_acc8(dy, x, q8, sc, seed=1, offset=i)
    elif which == "requant":
        # the benchmark size (8192 x 2048), then 4 and 16 times as many rows: steady state against launch cost
        for rows in (8192, 4 * 8192, 16 * 8192):
            N, K = rows, 2048
            for i in range(launches if rows == 8192 else 4):
                p, s, z = synth_w4(N, K, 10 + i, device)
                g = (torch.randn(N, K, device=device) * 1e-3).to(torch.bfloat16)
                o.requant_sr(p, s, z, g, 1e-4, (N, K), seed=7, offset=i)
                del p, s, z, g
    elif which == "gradq8":
        N, K = FFN, HID
        for i in range(launches):
            dw = (torch.randn(N, K, device=device) * 1e-3).to(torch.bfloat16)
            q8 = torch.empty((N, K), dtype=torch.int8, device=device)
            sc = torch.empty((N, 1), dtype=torch.bfloat16, device=device)
            o.gradq8_quant(dw, q8, sc, False, seed=1, offset=i)
            o.gradq8_quant(dw, q8, sc, True, seed=1, offset=i + 100)
    elif which == "ceiling":
        blk = MLPBlock(device)
        h = torch.randn(TOKENS, FFN, device=device).to(torch.bfloat16)
        print(json.dumps(bench_ceiling(device, blk, h)))
    elif which == "latent":
        N, K = 8192, 2048
        curve = (2, 0.125, 2, 0.25, 4)
        for i in range(launches):
            p, s, z = synth_w4(N, K, 40 + i, device)
            res = torch.randint(-2 ** 31, 2 ** 31 - 1, (N * K // 8,), device=device, dtype=torch.int64).to(torch.int32)
            lat = o.latent_w4_reconstruct(p, s, z, res, (N, K), *curve)
            o.latent_w4_requant(lat, s, z, res, (N, K), *curve)
    elif which == "adam8":
        N, K = 8192, 2048
        n, nblk = N * K, N * K // 2048
        curve = (2, 0.1875, 3, 0.375, 3)
        for i in range(launches):
            # fresh buffers per launch, so that every launch reads its operands from HBM
            p, s, z = synth_w4(N, K, 60 + i, device)
            res = torch.randint(-2 ** 31, 2 ** 31 - 1, (n // 8,), device=device, dtype=torch.int64).to(torch.int32)
            grad = (torch.randn(n, device=device) * 1e-3).to(torch.bfloat16)
            param = (torch.randn(n, device=device) * 0.02).to(torch.bfloat16)
            s1 = torch.randint(0, 256, (n,), device=device, dtype=torch.uint8)
            s2 = torch.randint(0, 256, (n,), device=device, dtype=torch.uint8)
            q = [torch.full((nblk, 1), v, device=device) for v in (1e-5, 1.3e-3, 1e-5, 2.6e-3)]
            o.adam8_update(grad, s1, s2, q[0], q[1], q[2], q[3], 0.9, 0.95, 1e-8, 1e-3, param=param)
            o.adam8_latent_w4_step(grad, p, res, s.view(-1), z.view(-1), (N, K), s1, s2, q[0], q[1], q[2], q[3], curve, curve,
                                   0.9, 0.95, 1e-8, 1e-3)
            w8 = torch.randint(-128, 128, (N, K), device=device, dtype=torch.int8)
            qs = ((torch.randn(N, device=device) * 0.01).abs() + 1e-3).to(torch.bfloat16)
            o.adam8_latent_w8_step(grad, w8, res, qs, s1, s2, q[0], q[1], q[2], q[3], curve, curve, 0.9, 0.95, 1e-8, 1e-3)
    elif which == "gemv":
        for (N, K) in [(4096, 4096), (11008, 4096), (4096, 11008)]:
            for M in (1, 4, 16):
                x = torch.randn(M, K, device=device).to(torch.bfloat16)
                for i in range(launches):
                    w = synth_w4(N, K, 20 + i, device)
                    o.a16w4_forward(x, *w, (N, K))
        # the fused gate / up product as one GEMV pass over both matrices
        for M in (1, 16):
            x = torch.randn(M, HID, device=device).to(torch.bfloat16)
            for i in range(launches):
                wg, wu = synth_w4(FFN, HID, 50 + i, device), synth_w4(FFN, HID, 70 + i, device)
                o.a16w4_gate_up_silu(x, wg, wu, (FFN, HID))
    elif which == "a8w8":
        for (N, K) in [(2048, 2048), (8192, 2048), (2048, 8192)]:
            x8 = torch.randint(-127, 128, (TOKENS, K), device=device, dtype=torch.int8)
            w8 = torch.randint(-127, 128, (N, K), device=device, dtype=torch.int8)
            sx = (torch.randn(TOKENS, device=device) * 0.05).abs()
            sw = (torch.randn(N, device=device) * 0.01).abs()
            for _ in range(launches):
                o.a8w8_forward(x8, w8, sx, sw)
    torch.cuda.synchronize()


def _cpu_time(fn, budget_s, min_runs=1, max_runs=7):
    """Median seconds per call after one warm-up, within a time budget."""
    fn()
    ts, t_start = [], time.time()
    while len(ts) < min_runs or (time.time() - t_start < budget_s and len(ts) < max_runs):
        t0 = time.time()
        fn()
        ts.append(time.time() - t0)
    ts.sort()
    return ts[len(ts) // 2], len(ts)


def cpu_baseline():
    """The reference's CPU path (nibble unpack -> bf16 group dequant -> bf16 torch.mm), restated in
    oracle/torch_ref.py, and the requant oracle (oracle/lq_oracle.c), on the host cores: the whole MLP
    step at 2048 tokens (the headline workload), and bounded samples of the OPT-125m layer (fwd + dX),
    the requantizer at its benchmark size and the decode shapes."""
    import numpy as np
    from oracle import c_oracle as co
    from oracle import torch_ref as tr
    from tests.util import bits
    os_cores = os.cpu_count() or 1
    cores = min(os_cores, 16)  # the box's share of the host; OMP_NUM_THREADS is set to the same there
    torch.set_num_threads(cores)
    gate = [t.cpu() for t in synth_w4(FFN, HID, 1, "cpu")] + [(FFN, HID)]
    up = [t.cpu() for t in synth_w4(FFN, HID, 2, "cpu")] + [(FFN, HID)]
    down = [t.cpu() for t in synth_w4(HID, FFN, 3, "cpu")] + [(HID, FFN)]
    g = torch.Generator().manual_seed(4)
    x = torch.randn(TOKENS, HID, generator=g).to(torch.bfloat16)
    dy = torch.randn(TOKENS, HID, generator=g).to(torch.bfloat16)

    def step():
        y, (gg, uu, h) = tr.llama_mlp_forward(x, gate, up, down)
        dh = dy.mm(tr.dequant_4bit_g(*down))
        du = dh * torch.nn.functional.silu(gg)
        dg = torch.ops.aten.silu_backward(dh * uu, gg)
        dx = dg.mm(tr.dequant_4bit_g(*gate)) + du.mm(tr.dequant_4bit_g(*up))
        return y, dx

    sec, runs = _cpu_time(step, 8.0, min_runs=3, max_runs=10)
    out = {"value": MLP_FLOP / sec / 1e12, "unit": "TFLOP/s", "cores": cores, "os_cpu_count": os_cores,
           "torch_num_threads": torch.get_num_threads(), "kind": "port",
           "sample": f"whole workload ({TOKENS} tokens, fwd + dX of the MLP block), 1 warm-up + {runs} timed runs (median), "
                     f"torch {torch.__version__} CPU bf16 mm, {sec:.2f} s per step",
           "cpu": _cpu_model()}
    # configs[0]: OPT-125m fc1 (3072 x 768) at 1024 tokens, forward + dX
    N0, K0, M0 = 3072, 768, 1024
    w0 = [t.cpu() for t in synth_w4(N0, K0, 5, "cpu")]
    x0 = torch.randn(M0, K0, generator=g).to(torch.bfloat16)
    dy0 = torch.randn(M0, N0, generator=g).to(torch.bfloat16)

    def c0():
        y = tr.w4_forward(x0, *w0, (N0, K0))
        dx = dy0.mm(tr.dequant_4bit_g(*w0, (N0, K0)))
        return y, dx
    sec, runs = _cpu_time(c0, 2.0, min_runs=3)
    out["c0"] = {"workload": "configs[0]: 3072x768 at 1024 tokens, fwd + dX", "TFLOP/s": 2 * 2 * M0 * N0 * K0 / sec / 1e12,
                 "ms": sec * 1e3, "runs": runs}
    # configs[1]: the requantizer at 8192 x 2048 (C oracle, OpenMP over the same cores)
    N1, K1 = 8192, 2048
    p1, s1, z1 = [t.cpu() for t in synth_w4(N1, K1, 10, "cpu")]
    g1 = (torch.randn(N1, K1, generator=g) * 1e-3).to(torch.bfloat16)
    a1 = (p1.numpy().view(np.uint8), bits(s1), bits(z1), bits(g1))
    sec, runs = _cpu_time(lambda: co.requant(*a1, 1e-4, N1, K1, seed=7, offset=0), 3.0, min_runs=3)
    nbytes = N1 * K1 // 2 * 2 + N1 * K1 * 2 + 4 * N1 * K1 // GROUP
    out["c1"] = {"workload": "configs[1]: requant 8192x2048, Philox mode, C oracle", "GB/s": nbytes / sec / 1e9, "ms": sec * 1e3,
                 "runs": runs, "omp_threads": os.environ.get("OMP_NUM_THREADS", "unset")}
    # configs[4]: decode shapes, the reference's dequantise-then-mm path
    c4 = []
    for (N, K) in [(4096, 4096), (11008, 4096), (4096, 11008)]:
        w = [t.cpu() for t in synth_w4(N, K, 20, "cpu")]
        for M in (1, 4, 16):
            xm = torch.randn(M, K, generator=g).to(torch.bfloat16)
            sec, runs = _cpu_time(lambda: tr.w4_forward(xm, *w, (N, K)), 0.6, min_runs=1, max_runs=3)
            nb = N * K // 2 + 4 * N * K // GROUP + 2 * M * K + 2 * M * N
            c4.append({"N": N, "K": K, "M": M, "ms": sec * 1e3, "GB/s": nb / sec / 1e9})
    out["c4"] = c4
    out["c4_note"] = "1 warm-up + 1-3 timed runs per point within 0.6 s each (a stated baseline, not a precise timing)"
    # configs[3]: the int8 GEMM with its scale epilogue (C oracle, OpenMP over the same cores; the reference's own
    # kernel for it is CUDA-only), once per shape on the first 256 of the 2048 tokens
    c3 = []
    rng = np.random.default_rng(3)
    Ms = 256
    for (N, K) in [(2048, 2048), (8192, 2048), (2048, 8192)]:
        x8 = rng.integers(-127, 128, (Ms, K), dtype=np.int8)
        w8 = rng.integers(-127, 128, (N, K), dtype=np.int8)
        sxv = np.abs(rng.standard_normal(Ms).astype(np.float32)) * 0.05
        swv = np.abs(rng.standard_normal(N).astype(np.float32)) * 0.01
        t0 = time.time()
        co.a8w8(x8, w8, sxv, swv, None, Ms, N, K)
        sec = time.time() - t0
        c3.append({"M_sample": Ms, "N": N, "K": K, "ms": sec * 1e3, "TOP/s": 2.0 * Ms * N * K / sec / 1e12})
    out["c3"] = c3
    out["c3_note"] = f"configs[3] shapes on a sample of {Ms} of the {TOKENS} tokens, one run each, int32 accumulate + fp32 scale epilogue"
    return out


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--settle-ms", type=float, default=150.0, help="untimed steps run for at least this long before the warm-up")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-mlp", action="store_true", help="skip the side measurements (requant, GEMV, A8W8)")
    ap.add_argument("--profile-target", choices=["gemm", "requant", "gemv", "a8w8", "latent", "adam8", "gradq8", "dw", "ceiling"],
                    help="run only a short fixed launch sequence of one kernel family (for rocprofv3); prints nothing except for 'ceiling'")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (no sharding, no collectives); use --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP kernels have no CPU fallback")
    from latentq_llm_amd import _C
    _C.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.profile_target:
        profile_target(dev, args.profile_target)
        return

    blk = MLPBlock(dev)
    # Settle the clock first: after an idle period the device takes tens of milliseconds of load to reach the
    # clock it sustains (a step timed in the first milliseconds reads ~5-10 % low), so run untimed steps for
    # at least --settle-ms, then the --warmup steps asked for.
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for _ in range(5):
            blk.step()
        torch.cuda.synchronize()
    settle_ms = (time.perf_counter() - t_settle) * 1e3
    for _ in range(args.warmup):
        blk.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        blk.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    value = MLP_FLOP / dt / 1e12

    # Dominant kernel: the dequant-GEMM. Per-launch duration of the step's four launches from HIP events on the
    # launch stream (the gate / up launches hold two products each: 2 x 184.68 GFLOP).
    o = blk.ops
    one = 2 * TOKENS * HID * FFN
    h, g, u = o.a16w4_gate_up_silu(blk.x, blk.gate, blk.up, (FFN, HID), save=True)
    dg, du = o.a16w4_dx_silu_bwd(blk.dy, *blk.down, (HID, FFN), g, u)
    dxb = torch.empty((TOKENS, HID), dtype=torch.bfloat16, device=dev)
    kern = {}
    for name, fn, fl in [
        ("fwd_gate_up_silu", lambda: o.a16w4_gate_up_silu(blk.x, blk.gate, blk.up, (FFN, HID), save=True), 2 * one),
        ("fwd_down", lambda: o.a16w4_forward(h, *blk.down, (HID, FFN)), one),
        ("dx_down_silu_bwd", lambda: o.a16w4_dx_silu_bwd(blk.dy, *blk.down, (HID, FFN), g, u), one),
        ("dx_gate_up_pair", lambda: o.a16w4_dx_pair(dg, blk.gate, du, blk.up, (FFN, HID), out=dxb), 2 * one),
        # the same products as separate launches with a plain store (what the layers run on their own)
        ("fwd_gate_or_up", lambda: o.a16w4_forward(blk.x, *blk.gate, (FFN, HID)), one),
        ("dx_down", lambda: o.a16w4_dx(blk.dy, *blk.down, (HID, FFN)), one),
        ("dx_gate", lambda: o.a16w4_dx(dg, *blk.gate, (FFN, HID), out=dxb), one),
        ("dx_up_acc", lambda: o.a16w4_dx(du, *blk.up, (FFN, HID), out=dxb, accumulate=True), one),
    ]:
        sec = event_time(fn, 50)
        kern[name] = {"us": sec * 1e6, "GFLOP": fl / 1e9, "TFLOP/s": fl / sec / 1e12, "frac_mfma_bf16": fl / sec / PEAK_BF16}
    # The same four launches timed inside the step, where each finds its operands as the previous launch left them
    # (g and u come from HBM there, not from the last-level cache as in a loop over one launch): 40 steps with events
    # between the launches, after 10 untimed ones. The roofline figure uses these.
    for _ in range(10):
        blk.step()
    evs = [blk.step_events() for _ in range(40)]
    torch.cuda.synchronize()
    for j, name in enumerate(PMC_LAUNCHES):
        us = sum(e[j].elapsed_time(e[j + 1]) for e in evs) / len(evs) * 1e3
        kern[name]["isolated_us"] = kern[name]["us"]
        kern[name]["us"] = us
        kern[name]["TFLOP/s"] = kern[name]["GFLOP"] * 1e9 / (us * 1e-6) / 1e12
        kern[name]["frac_mfma_bf16"] = kern[name]["GFLOP"] * 1e9 / (us * 1e-6) / PEAK_BF16
    del evs
    tot = sum(kern[k]["us"] for k in PMC_LAUNCHES)
    # per 184.68 GFLOP product: six of them in the four launches
    avg_us = tot / 6
    achieved = one / (avg_us * 1e-6) / 1e12
    roofline = {"bound": "mfma", "kernel": "A16W4 dequant-GEMM: gemm_fwd_direct_kernel<2, *> (forward), gemm_kernel<1> (dX)",
                "achieved": achieved, "peak": PEAK_BF16 / 1e12, "unit": "TFLOP/s", "frac": achieved * 1e12 / PEAK_BF16,
                "avg_launch_us": avg_us, "flop_per_launch": one,
                "note": "per product of 2*2048*4096*11008 flop: total time of the step's four GEMM launches, each timed with HIP events inside the step, / 6 (the two gate/up launches hold two each)",
                "traffic": gemm_traffic_bytes(),
                "traffic_unit": "HBM bytes per product: the four launches' rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated on a copy, / 6"}
    # the step with the glue as tensor-library kernels, for comparison
    for _ in range(20):
        blk.step_unfused()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(50):
        blk.step_unfused()
    torch.cuda.synchronize()
    unfused_ms = (time.perf_counter() - t0) / 50 * 1e3
    del g, u, dg, du, dxb

    line = {
        "metric": "A16W4 GEMM TFLOP/s (7B MLP, 2048 tok)", "value": value, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_ms": settle_ms, "ms_per_step": dt * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "configs[2]: A16W4 Llama-2-7B MLP block, 4x512=2048 bf16 tokens, forward + dX "
                               "through gate/up (11008x4096) and down (4096x11008), int4 group 128",
                   "tokens": TOKENS, "flop_per_step": MLP_FLOP},
        "roofline": roofline,
        "gemm_kernels": kern,
        "step_layer_by_layer": {"ms_per_step": unfused_ms, "TFLOP/s": MLP_FLOP / (unfused_ms * 1e-3) / 1e12,
                                "what": "six GEMM launches + six bf16 tensor-library kernels (silu, three products, silu backward, add)"},
    }
    if not args.only_mlp:
        ceil = bench_ceiling(dev, blk, h)
        loop = ceil["mfma_loop_random_operands_2wg_per_cu"]["TFLOP/s"]
        roofline["ceiling"] = {"what": "MFMA-only loop (lq_calib_mfma_loop), random bf16 operands, the forward kernel's 2 x 4 waves per compute unit",
                               "TFLOP/s": loop, "achieved_over_ceiling": achieved / loop}
        line["ceiling"] = ceil
        line["gate_up_silu"] = bench_gate_up(dev, blk)
        del blk
        torch.cuda.empty_cache()
        line["c0"] = bench_c0(dev)
        line["requant"] = bench_requant(dev)
        line["gradq8"] = bench_gradq8(dev)
        line["latent_lbit4"] = bench_latent(dev)
        line["gemv"] = bench_gemv(dev)
        line["a8w8"] = bench_a8w8(dev)
        line["a8w8_layer_step"] = bench_a8w8_layer_step(dev)
        line["adam8"] = bench_adam8(dev)
        line["dw"] = bench_dw(dev)
        line["hbm_copy"] = bench_copy(dev)
    line["cpu_baseline"] = None if args.no_cpu else cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()

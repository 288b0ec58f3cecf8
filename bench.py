#!/usr/bin/env python3
"""Headline benchmark: HOT linear-layer backward, microseconds per layer.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

One step = one pass of the fused backward (hot_linear_backward through the C
ABI) over one batch of synthetic input already resident in HBM: the ViT-B fc1
layer at batch 64 x 197 tokens (L = 12608, O = 3072, I = 768), bf16 g_y / W,
INT4 Hadamard-quantised g_x GEMM, Hadamard low-rank (n = 64, r = 36) INT8 g_W
GEMM, round-to-nearest, per-tensor steps, with the INT8 activation buffer
written beforehand by the forward-side kernel.  Four input sets (> 256 MiB in
total) are rotated so that g_y is not served from the Infinity Cache.

Prints ONE JSON line.  Besides the contract fields it carries
  roofline      the dominant kernel of the step, timed live inside the fused
                step with HIP events on the launch stream
                (hot_linear_backward_kernels), against the chip's published peak
  cpu_baseline  the op-for-op CPU port of the reference's fake-quant path
                (oracle/fakequant_port.py) on the same layer, on the host cores
  ceilings      what this box reaches with a plain copy kernel and a loop of INT8 MFMAs
  kernels       per-kernel microseconds and achieved rates for this layer
  layers        the same step at every ViT-B and Llama-7B layer shape, bf16 and fp32
  llama_gate_up per-kernel pass at the Llama-7B gate/up shape
  llama_gate_up_python_rule  the same layer with the reference's own low-rank rule (n = 8192, r = 2080)
  hq_rowwise_sweep  the row-wise quantise kernel alone over the kernel-level sweep (launches replayed
                from a HIP graph, so no host time is in the figures)
  quantiser_grid the step over bits x rounding x step granularity x low-rank setting
  measure_py    the reference's latency harness (cuda_measure/measure.py) on the drop-in op
  vit_b16       whole-model backward with every layer swapped
  forward_gemm  the plain bf16 forward product at the layer shapes: vendor library beside hot_gemm_bf16
  schemes       the layer's backward under every transform scheme / quantiser family the native path runs
  host_cost     host microseconds of one backward call (C entry point, Python op), one- and two-stream order
This run uses one GPU; --gpus above 1 is refused.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0      # MI355X dense INT8 MFMA, published


def _events(fn, iters, warm):
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters     # microseconds per call


def make_layer(L, O, I, dtype, dev, nsets, seed=0):
    """Synthetic inputs of the GPU benchmark workloads: x ~ N(0,1); g_y ~ N(0, 1e-3) with
    1 % of the entries x50; W uniform(+-1/sqrt(I)) (kaiming-uniform)."""
    import torch
    g = torch.Generator(device=dev).manual_seed(seed)
    w = ((torch.rand(O, I, generator=g, device=dev) * 2 - 1) / I ** 0.5).to(dtype)
    sets = []
    for _ in range(nsets):
        x = torch.randn(L, I, generator=g, device=dev).to(dtype)
        gy = torch.randn(L, O, generator=g, device=dev) * 1e-3
        gy = torch.where(torch.rand(L, O, generator=g, device=dev) < 0.01, gy * 50, gy).to(dtype)
        sets.append((x, gy))
    return w, sets


def profiled_traffic(workload="vit_b_fc1"):
    """HBM bytes per launch of the kernels of the step at a workload ("vit_b_fc1", "llama_gate_up"), as
    the committed counter summary gives them (profiles/hot_linear_backward_<workload>_bf16.hbm_traffic.txt:
    lines `traffic_bytes <kernel key> <bytes>` and `measured_at <commit>`), or (None, None) when the
    summary is absent or carries no such lines.  The figures belong to the commit named there: kernels
    changed since then are listed without traffic."""
    path = os.path.join(ROOT, "profiles", "hot_linear_backward_%s_bf16.hbm_traffic.txt" % workload)
    table, commit = {}, None
    try:
        for line in open(path):
            f = line.split()
            if len(f) == 3 and f[0] == "traffic_bytes":
                table[f[1]] = float(f[2])
            elif len(f) >= 2 and f[0] == "measured_at":
                commit = f[1]
    except OSError:
        return None, None
    return (table or None), commit


GEMM_VARIANT_NAMES = {1: "gemm_i8_pipe_kernel<128x128, 3 stages>", 2: "gemm_i8_pipe_kernel<128x128, 4 stages>",
                      3: "gemm_i8_pipe_kernel<256x256, 4 stages>", 4: "gemm_i8_kernel<128x128, register-staged>",
                      5: "gemm_i8_pipe_kernel<128x128, split K>", 6: "gemm_i8_slot_kernel<256x256>",
                      7: "gemm_i8_slot_kernel<128x128>", 8: "gemm_i8_slot_kernel<160x256>",
                      9: "gemm_i8_slot_kernel<96x128>", 10: "gemm_i8_slot_kernel<64x128>", 11: "gemm_i8_slot_kernel<32x128>"}


def gemm_kernel_name(M, N, K, bits, with_ws=False):
    from hot_amd import ops
    return GEMM_VARIANT_NAMES.get(ops.gemm_plan(M, N, K, bits, workspace_bytes=(1 << 40) if with_ws else 0), "gemm")


def kernel_table(w, sets, bufs, opt, ws, iters, warm, traffic=None):
    """Per-kernel durations INSIDE the fused step: hot_linear_backward_kernels records a HIP event
    on the launch stream after every kernel; the table prices each kernel with its algorithmic
    bytes (sizeof(in) read once + codes written) or operations (2 M N K)."""
    import torch
    from hot_amd import ops
    L, O = sets[0][1].shape
    I = w.shape[1]
    e = sets[0][1].element_size()
    lp = opt.lprime(L)
    from hot_amd import _lib
    gx_splits = int(_lib.lib().hot_gemm_splits(L, I, O, opt.gx_bits))
    gw_splits = int(_lib.lib().hot_gemm_splits(O, I, lp, 8))
    acc = [0.0] * 8
    for it in range(warm + iters):
        i = it % len(sets)
        _, _, t = ops.linear_backward(sets[i][1], w, bufs[i][0], bufs[i][1], opt, timing="kernels", workspace=ws)
        if it >= warm:
            acc = [a + b for a, b in zip(acc, t)]
    us = [a / iters * 1e6 for a in acc]
    spec = [
        ("clear", "hot::clear3_kernel", us[0], "hbm", 0.0),
        ("gy_stats", "hot::colwise_kernel<.., PASS 0, RS 16> (g_y: token-wise + row-wise absmax)", us[1], "hbm", L * O * e),
        ("gy_hla_quant", "hot::colwise_kernel<.., PASS 1> (g_y: HLA + INT8, transposed)", us[2], "hbm", L * O * e + lp * O),
        ("gy_hq_quant", "hot::hq_tensor_kernel (g_y: Hadamard-16 + INT%d)" % opt.gx_bits, us[3], "hbm",
         L * O * e + L * O * opt.gx_bits // 8),
        ("w_stats", "hot::colwise_kernel<.., PASS 0> (W)", us[4], "hbm", O * I * e),
        ("w_quant", "hot::colwise_kernel<.., PASS 1> (W: Hadamard-16 + INT%d, transposed)" % opt.w_bits, us[5], "hbm",
         O * I * e + O * I * opt.w_bits // 8),
        ("gemm_gx", "hot::%s INT%d (g_x)" % (gemm_kernel_name(L, I, O, opt.gx_bits), opt.gx_bits), us[6], "mfma", 2.0 * L * O * I),
        ("gemm_gw", "hot::%s INT8 (g_W)" % gemm_kernel_name(O, I, lp, 8, with_ws=True)
         + (" in %d K ranges + gemm_i8_reduce_kernel" % gw_splits if gw_splits > 1 else ""), us[7], "mfma", 2.0 * O * I * lp),
    ]
    launches = {"gemm_gw": 2 if gw_splits > 1 else 1, "gemm_gx": 2 if gx_splits > 1 else 1}
    rows = []
    for key, name, t, bound, alg in spec:
        peak = HBM_PEAK_GBS if bound == "hbm" else INT8_PEAK_TOPS
        ach = (alg / t / 1e3 if bound == "hbm" else alg / t / 1e6) if t > 0 else 0.0      # GB/s | TOP/s
        rows.append(dict(key=key, kernel=name, us=round(t, 2), bound=bound, achieved=round(ach, 1), peak=peak,
                         unit="GB/s" if bound == "hbm" else "TOP/s", frac=round(ach / peak, 4),
                         traffic=(round(traffic[key]) if traffic and key in traffic else None),
                         work=("%.0f bytes" % alg if bound == "hbm" else "%.0f ops" % alg),
                         launches=launches.get(key, 1)))
    return rows


def gemm_launch_times(w, sets, bufs, opt, iters=20, warm=4):
    """Average launch duration of the two GEMM kernels of the step, each timed over `iters`
    back-to-back launches between two HIP events on the launch stream, on the step's real
    operands (produced by the transform kernels), rotating the input sets."""
    import torch
    from hot_amd import ops
    L, O = sets[0][1].shape
    I = w.shape[1]
    lp = opt.lprime(L)
    qw, sw = ops.wq_colwise(w, n=opt.n_o, bits=opt.w_bits, rounding=opt.w_round, scale=opt.w_scale)
    gx_ops, gw_ops = [], []
    for (x, gy), (xq, sx) in zip(sets, bufs):
        qg, sg = ops.hq_rowwise(gy, n=opt.n_o, bits=opt.gx_bits, rounding=opt.gx_round, scale=opt.gx_scale)
        if qg.shape[1] != qw.shape[1]:       # O not a multiple of the K tile: pad the packed g_y codes
            pad = torch.zeros((L, qw.shape[1]), dtype=torch.int8, device=gy.device)
            pad[:, :qg.shape[1]] = qg
            qg = pad
        qgp, sgp, _ = ops.hla_tokenwise(gy, opt.hla_n, opt.hla_rows, bits=opt.gw_bits, rounding=opt.gw_round,
                                        scale=opt.gw_scale)
        gx_ops.append((qg, sg))
        gw_ops.append((qgp, sgp, xq, sx))
    state = {"i": 0}

    def run_gx():
        qg, sg = gx_ops[state["i"] % len(gx_ops)]
        state["i"] += 1
        ops.gemm_i8(qg, qw, O, opt.gx_bits, sg, sw, 1.0 / opt.n_o, out_dtype=sets[0][1].dtype)

    def run_gw():
        qgp, sgp, xq, sx = gw_ops[state["i"] % len(gw_ops)]
        state["i"] += 1
        ops.gemm_i8(qgp, xq, lp, 8, sgp, sx, 1.0 / opt.hla_n, out_dtype=sets[0][1].dtype)

    return _events(run_gx, iters, warm), _events(run_gw, iters, warm)


def step_time(w, sets, opt, steps, warmup):
    import torch
    from hot_amd import ops
    bufs = [ops.abc_forward(x, opt) for (x, _) in sets]
    ws = None
    state = {"i": 0}

    def one():
        i = state["i"] % len(sets)
        state["i"] += 1
        ops.linear_backward(sets[i][1], w, bufs[i][0], bufs[i][1], opt, workspace=ws)

    # one allocation of the workspace outside the timed region
    import ctypes as C
    from hot_amd import _lib
    L, O = sets[0][1].shape
    need = _lib.lib().hot_backward_workspace_bytes(L, O, w.shape[1], C.byref(opt.to_c()))
    ws = torch.empty(need, dtype=torch.uint8, device=w.device)
    for _ in range(warmup):
        one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps, bufs, ws


def cpu_baseline(reps=5):
    """The reference's CPU path for this layer, restated op for op (dense
    matmul transforms, float fake quantisation), fp32, on the host cores."""
    import torch
    from oracle import fakequant_port as fq
    L, O, I = 12608, 3072, 768
    x, w, gy = fq.config1_inputs(L, O, I, seed=0)
    h_out, h_bs = fq.matrices(L, O)
    cfg = fq.PortConfig()
    xq, sx = fq.setup_context(x, h_bs, cfg)
    fq.backward(gy, w, xq, sx, h_out, h_bs, cfg)       # warm-up
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fq.backward(gy, w, xq, sx, h_out, h_bs, cfg)
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return dict(value=round(ts[len(ts) // 2] * 1e6, 1), unit="us/layer", cores=torch.get_num_threads(),
                kind="port", sample="whole layer (L=12608 O=3072 I=768 fp32, int quantisers 4/4/8/8, "
                                    "HLA n=64 r=36), median of %d repetitions after 1 warm-up" % reps,
                host_cpus=os.cpu_count())


def hq_rowwise_sweep(dev, reps=20):
    """Kernel-level extra: the fused block-Hadamard + per-token absmax step + quantise kernel alone
    (hot_hq_rowwise, bf16 input with per-channel scales drawn log-uniform in [0.1, 10]), GB/s of
    algorithmic bytes (input read once + codes + steps written) against the 8 TB/s HBM peak.  `reps`
    launches are captured into a HIP graph once and replayed between two events, so the figures hold
    no host-side launch time; two input tensors alternate inside the graph."""
    import torch
    from hot_amd import _lib, ops
    lib = _lib.lib()
    rows = []
    g = torch.Generator(device=dev).manual_seed(0)
    side = torch.cuda.Stream()
    for M in (4096, 16384, 65536):
        for K in (768, 3072, 4096, 11008):
            xs = [(torch.randn(M, K, generator=g, device=dev) *
                   (10.0 ** (torch.rand(K, generator=g, device=dev) * 2 - 1))).to(torch.bfloat16) for _ in range(2)]
            scales = torch.empty(M, dtype=torch.float32, device=dev)
            for n in (16, 32, 64):
                if K % n:
                    continue
                for bits in (4, 8):
                    codes = torch.empty((M, K * bits // 8), dtype=torch.int8, device=dev)

                    def launch(i, stream):
                        _lib.check(lib.hot_hq_rowwise(xs[i & 1].data_ptr(), _lib.BF16, M, K, n, bits, ops.ROUND_NEAREST, 0, 0,
                                                      ops.SCALE_ROW, codes.data_ptr(), scales.data_ptr(), None, 0, stream))
                    torch.cuda.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.stream(side):
                        launch(0, side.cuda_stream)
                        side.synchronize()
                        with torch.cuda.graph(graph, stream=side):
                            for i in range(reps):
                                launch(i, side.cuda_stream)
                        graph.replay()
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        e0.record(side)
                        graph.replay()
                        e1.record(side)
                        side.synchronize()
                    us = e0.elapsed_time(e1) * 1e3 / reps
                    byt = M * K * 2 + M * K * bits // 8 + 4 * M
                    rows.append([M, K, n, bits, round(us, 2), round(byt / us / 1e3), round(byt / us / 1e3 / HBM_PEAK_GBS, 3)])
                    del graph
            del xs
    return {"columns": ["M", "K", "hadamard_block", "bits", "us", "GB/s", "frac_of_8TB/s"], "rows": rows,
            "note": "per-token steps, round-to-nearest; %d launches replayed from a HIP graph between two events" % reps}


def layer_table(dev, steps=30, warmup=8):
    """The step at every layer shape of the ViT-B (batch 64 x 197 tokens, make_WHT rule: n 64, r 36) and
    Llama-7B (8192 tokens, n 16 / 8 lowest sequencies) configurations, bf16 and fp32, per-tensor steps,
    round-to-nearest, INT4 g_x / INT8 g_W; beside it the two plain matmuls (g_y @ W, g_y^T @ x) in the
    same dtype through torch (hipBLASLt), and the forward-side buffer write."""
    import torch
    from hot_amd import ops
    from hot_amd.hadamard_matmul import hla_rows, paper_rows
    shapes = [("vit_qkv", 12608, 2304, 768), ("vit_proj", 12608, 768, 768), ("vit_fc1", 12608, 3072, 768),
              ("vit_fc2", 12608, 768, 3072), ("llama_qkvo", 8192, 4096, 4096), ("llama_gate_up", 8192, 11008, 4096),
              ("llama_down", 8192, 4096, 11008)]
    rows = []
    for name, L, O, I in shapes:
        n, sel = hla_rows(L) if name.startswith("vit") else paper_rows(16, 8)
        opt = ops.HotOptions(n_o=16, hla_n=int(n), hla_rows=tuple(int(v) for v in sel))
        for dt, dname in ((torch.bfloat16, "bf16"), (torch.float32, "fp32")):
            w, sets = make_layer(L, O, I, dt, dev, nsets=3 if name.startswith("vit") else 2, seed=3)
            sec, bufs, ws = step_time(w, sets, opt, steps, warmup)
            st = {"i": 0}

            def mm():
                x, gy = sets[st["i"] % len(sets)]
                st["i"] += 1
                torch.matmul(gy, w)
                torch.matmul(gy.t(), x)

            def fwd():
                x, _ = sets[st["i"] % len(sets)]
                st["i"] += 1
                ops.abc_forward(x, opt)
            rows.append([name, L, O, I, "n=%d r=%d" % (opt.hla_n, opt.hla_r), dname, round(sec * 1e6, 1),
                         round(_events(mm, 10, 3), 1), round(_events(fwd, 10, 3), 1)])
            del w, sets, bufs, ws
            torch.cuda.empty_cache()
    return {"columns": ["layer", "L", "O", "I", "hla", "dtype", "hot_backward_us", "two_matmuls_us", "buffer_write_us"],
            "rows": rows, "note": "%d steps after %d warm-ups, inputs rotated" % (steps, warmup)}


def forward_gemm_table(dev):
    """The plain bf16 linear layer y = x W^T + b (utils/quant_matmul.py:173-176) at the layer shapes:
    torch's F.linear (the vendor library) beside hot_gemm_bf16, the same product through the data path
    of this library's integer kernels.  Decides whether the forward product is worth owning (it would
    have to be, for the activation buffer's statistics pass to move into its prologue)."""
    import torch
    import torch.nn.functional as F
    from hot_amd import ops
    rows = []
    for name, L, O, I in (("vit_qkv", 12608, 2304, 768), ("vit_proj", 12608, 768, 768), ("vit_fc1", 12608, 3072, 768),
                          ("vit_fc2", 12608, 768, 3072), ("llama_gate_up", 8192, 11008, 4096), ("llama_down", 8192, 4096, 11008)):
        g = torch.Generator(device=dev).manual_seed(7)
        x = torch.randn(L, I, device=dev, generator=g).bfloat16()
        w = (torch.randn(O, I, device=dev, generator=g) * 0.03).bfloat16()
        b = torch.randn(O, device=dev, generator=g).bfloat16()
        vendor = _events(lambda: F.linear(x, w, b), 20, 5)
        own = _events(lambda: ops.gemm_bf16(x, w, b), 20, 5)
        rows.append([name, L, O, I, round(vendor, 1), round(own, 1), round(own / vendor, 2)])
        del x, w, b
    return {"columns": ["layer", "L", "O", "I", "vendor_us", "hot_gemm_bf16_us", "ratio"], "rows": rows,
            "note": "bf16, bias added in the epilogue of both; 20 calls after 5 warm-ups"}


def scheme_table(dev):
    """The layer's backward through autograd (HQ_Linear, ViT-B fc1, bf16, 2-D tokens) under every transform
    scheme and quantiser family the native path runs: the fused call for gih_gwlr / hadamard, the separate
    g_x entry points for the schemes that project g_y along the tokens and for the logarithmic quantiser
    (kept for completeness of the reference's scheme list, not tuned)."""
    import torch
    from hot_amd import args
    from hot_amd.quant_matmul import HQ_Linear
    L, O, I = 12608, 3072, 768
    saved = {k: getattr(args, k) for k in dir(args) if not k.startswith("_") and not callable(getattr(args, k))}
    rows = []
    try:
        for label, recipe in (("gih_gwlr int", dict()), ("gih_gwlr stoch per-token", dict(gx="nq", gw="nq")),
                              ("hadamard", dict(scheme="hadamard")), ("low_rank", dict(scheme="low_rank")),
                              ("gilr_gwh", dict(scheme="gilr_gwh")), ("gih_gwlr luq g_x", dict(gx="luq")),
                              ("gih_gwlr luq g_W", dict(gw="luq", gw_bits=4))):
            args.hot_recipe(**recipe)
            torch.manual_seed(0)
            lin = HQ_Linear(I, O, bias=False).to(dev).to(torch.bfloat16)
            x = torch.randn(L, I, device=dev, dtype=torch.bfloat16, requires_grad=True)
            gy = (torch.randn(L, O, device=dev) * 1e-3).to(torch.bfloat16)
            y = lin(x)
            us = _events(lambda: torch.autograd.grad(y, (x, lin.weight), gy, retain_graph=True), 20, 10)
            rows.append([label, round(us, 1)])
            del lin, x, gy, y
            torch.cuda.empty_cache()
    finally:
        for k, v in saved.items():
            setattr(args, k, v)
    return {"columns": ["scheme / quantisers", "backward_us"], "rows": rows,
            "note": "L=12608 O=3072 I=768 bf16; 20 backward passes of one saved forward after 10 warm-ups"}


def host_cost(dev, calls=300):
    """Host time of one backward call: the C entry point through ctypes with prepared arguments, and
    ops.linear_backward, at a shape whose kernels are short (64 tokens, O = I = 64), issued back to back
    without waiting for the GPU, in the one-stream order (what the library picks for short calls) and
    with the two-stream order forced (three event record / wait pairs more)."""
    import ctypes as C
    import time
    import torch
    from hot_amd import _lib, ops
    from hot_amd.hadamard_matmul import hla_rows
    L, O, I = 64, 64, 64
    n, rows = hla_rows(L)
    w, sets = make_layer(L, O, I, torch.bfloat16, dev, nsets=2, seed=5)
    out = {}
    for label, streams in (("one_stream", 1), ("two_streams", 2)):
        opt = ops.HotOptions(n_o=16, hla_n=int(n), hla_rows=tuple(int(v) for v in rows), streams=streams)
        bufs = [ops.abc_forward(x, opt) for (x, _) in sets]
        cfg = opt.to_c()
        need = _lib.lib().hot_backward_workspace_bytes(L, O, I, C.byref(cfg))
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        gx = torch.empty((L, I), dtype=torch.bfloat16, device=dev)
        gw = torch.empty((O, I), dtype=torch.bfloat16, device=dev)
        st = torch.cuda.current_stream().cuda_stream
        fn = _lib.lib().hot_linear_backward

        def c_call(i):
            gy = sets[i % 2][1]
            xq, sx = bufs[i % 2]
            fn(gy.data_ptr(), w.data_ptr(), 1, xq.data_ptr(), sx.data_ptr(), L, O, I, C.byref(cfg), gx.data_ptr(),
               gw.data_ptr(), 1, ws.data_ptr(), ws.numel(), None, st)

        def py_call(i):
            xq, sx = bufs[i % 2]
            ops.linear_backward(sets[i % 2][1], w, xq, sx, opt)

        for name, call in (("c_call_us", c_call), ("python_call_us", py_call)):
            for i in range(30):
                call(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(calls):
                call(i)
            t1 = time.perf_counter()
            torch.cuda.synchronize()
            out.setdefault(name, {})[label] = round((t1 - t0) / calls * 1e6, 1)
    out["note"] = "%d calls issued back to back, wall time of the issuing loop per call (the GPU drains afterwards)" % calls
    return out


def measure_py(dev, trials=100):
    """The reference's latency harness (cuda_measure/measure.py:35-80) on the drop-in op: L = 49 tokens,
    O = 3072, I = 768, lognormal(1, 0.1) inputs (numpy seed 2023), `trials` trials, medians.  As there:
    the plain pair of matmuls by wall clock with device synchronisation, the op by the sum of the stage
    times it returns (per-token and per-tensor steps); the op's wall clock is reported beside it."""
    import statistics
    import numpy as np
    import torch
    from hot_amd import HLQ_backward
    B, O, I = 49, 3072, 768
    rng = np.random.RandomState(2023)
    fp, tok, ten, tok_wall, ten_wall = [], [], [], [], []
    for _ in range(trials):
        X = torch.tensor(rng.lognormal(1.0, 0.1, B * I).reshape(B, I), dtype=torch.float32).to(dev)
        Go = torch.tensor(rng.lognormal(1.0, 0.1, B * O).reshape(B, O), dtype=torch.float32).to(dev)
        W = torch.tensor(rng.lognormal(1.0, 0.1, O * I).reshape(O, I), dtype=torch.float32).to(dev)
        torch.cuda.synchronize()
        t0 = time.time()
        torch.matmul(Go, W)
        torch.cuda.synchronize()
        torch.matmul(Go.T, X)
        torch.cuda.synchronize()
        fp.append(time.time() - t0)
        for per_token, acc, wall in ((True, tok, tok_wall), (False, ten, ten_wall)):
            t0 = time.time()
            _, _, tl = HLQ_backward.backward(Go, W, X, 0, 0, 16, per_token)
            torch.cuda.synchronize()
            wall.append(time.time() - t0)
            acc.append(sum(tl))
    med = lambda v: round(statistics.median(v) * 1e6, 1)
    return {"shape": {"L": B, "O": O, "I": I}, "trials": trials, "unit": "us (medians)",
            "fp_matmuls_wall": med(fp), "per_token_stage_sum": med(tok), "per_tensor_stage_sum": med(ten),
            "per_token_wall": med(tok_wall), "per_tensor_wall": med(ten_wall),
            "note": "stage sums are HIP-event times of the kernels run one after the other, as the op's time list "
                    "reports them; wall clock adds the Python and launch overhead of one call"}


def quantiser_grid(w, sets, steps=60, warmup=10):
    """Extra: the same step at the headline shape over the quantiser settings of the g_x path (bits x
    rounding x step granularity; the g_W path follows rounding and granularity at INT8) and the two
    low-rank settings; us per layer, inputs rotated as in the headline measurement."""
    from hot_amd import ops
    from hot_amd.hadamard_matmul import hla_rows, paper_rows
    L = sets[0][1].shape[0]
    rows = []
    for hla, (n, sel) in (("n=64 r=36", hla_rows(L)), ("n=16 r=8", paper_rows(16, 8))):
        for bits in (4, 8):
            for rnd, rname in ((ops.ROUND_NEAREST, "nearest"), (ops.ROUND_STOCH, "stochastic")):
                for sc, sname in ((ops.SCALE_TENSOR, "per-tensor"), (ops.SCALE_ROW, "per-token")):
                    opt = ops.HotOptions(n_o=16, hla_n=int(n), hla_rows=tuple(int(v) for v in sel), gx_bits=bits,
                                         w_bits=bits, gx_round=rnd, gw_round=rnd, gx_scale=sc, gw_scale=sc, seed=1)
                    sec, _, _ = step_time(w, sets, opt, steps, warmup)
                    rows.append([hla, bits, rname, sname, round(sec * 1e6, 1)])
    return {"columns": ["hla", "gx_bits", "rounding", "steps", "us_per_layer"], "rows": rows}


def vit_b16_backward(dev, batch=128, steps=3):
    """Whole-model extra: ViT-B/16 (hot_amd/vit.py, random weights, bf16) on synthetic images, every
    Linear / Conv2d swapped for the HOT layers, quantisers chosen per layer by the calibration pass;
    backward time of one step against the same model with plain layers (hipBLASLt bf16)."""
    import torch
    import torch.nn as nn
    from hot_amd import args, lqs
    from hot_amd import utils as hutils
    from hot_amd.quant_matmul import HQ_Conv2d, HQ_Linear
    from hot_amd.vit import ViT

    torch.manual_seed(0)
    model = ViT().to(dev).to(torch.bfloat16)
    img = torch.randn(batch, 3, 224, 224, device=dev, dtype=torch.bfloat16)
    tgt = torch.randint(0, 100, (batch,), device=dev)

    def backward_ms(m):
        """(backward, forward + backward) of one step, best of `steps` after one warm-up step"""
        best = best_all = None
        for it in range(steps + 1):
            m.zero_grad(set_to_none=True)
            torch.cuda.synchronize()
            ef, e0, e1 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
            ef.record()
            loss = nn.functional.cross_entropy(m(img).float(), tgt)
            e0.record()
            loss.backward()
            e1.record()
            torch.cuda.synchronize()
            if it > 0:
                ms, ms_all = e0.elapsed_time(e1), ef.elapsed_time(e1)
                best = ms if best is None else min(best, ms)
                best_all = ms_all if best_all is None else min(best_all, ms_all)
        return best, best_all

    plain, plain_all = backward_ms(model)
    saved = {k: getattr(args, k) for k in dir(args) if not k.startswith("_") and not callable(getattr(args, k))}
    try:
        args.hot_recipe(gx="stoch", gw="stoch")
        hutils.replace_layers(model, nn.Conv2d, HQ_Conv2d)
        hutils.replace_layers(model, nn.Linear, HQ_Linear)
        hutils.name_layers(model)
        args.batched_mode = "flatten"
        args.layer_quant_dict.clear()
        lqs.calibrate(model, [(img[:32], tgt[:32])], nn.CrossEntropyLoss())
        args.quantAuto = True
        hot, hot_all = backward_ms(model)
        picks = list(args.layer_quant_dict.values())
        # the reference's own treatment of 3-D activations: every sample a problem of its own (197
        # tokens: no block divides them, so no low-rank projection; one step per sample), one
        # library call per layer
        args.batched_mode = "per_sample"
        per_sample, _ = backward_ms(model)
    finally:
        for k, v in saved.items():
            setattr(args, k, v)
        args.layer_quant_dict.clear()
    return {"model": "ViT-B/16, batch %d, bf16, flattened tokens" % batch, "backward_ms_plain_bf16": round(plain, 2),
            "backward_ms_hot": round(hot, 2), "forward_backward_ms_plain_bf16": round(plain_all, 2),
            "forward_backward_ms_hot": round(hot_all, 2), "backward_ms_hot_per_sample_steps": round(per_sample, 2),
            "hot_layers": len(picks) // 2,
            "per_token_quantiser_layers": sum(1 for i, v in enumerate(picks) if i % 2 == 0 and v == "norm_quantizer")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the per-kernel table and the Llama shape")
    ap.add_argument("--table-only", action="store_true",
                    help="of the extras keep only the per-kernel table (kernels launched one after the other, as "
                         "the roofline entry measures them); the profiling runs use this")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 512 MiB device-to-device copies (a kernel of known traffic, for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--python-rule", action="store_true",
                    help="with --llama-table: the reference's own low-rank rule (n = 8192, r = 2080), the step only")
    ap.add_argument("--llama-table", action="store_true",
                    help="only the per-kernel pass at the Llama-7B gate/up shape (kernels launched one after the "
                         "other), printed as one JSON line; for profiling runs of that shape")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding)"
              % a.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from hot_amd import ops
    from hot_amd.hadamard_matmul import hla_rows, paper_rows
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if a.copy_calibration:
        src = torch.empty(512 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if a.llama_table:
        Ll, Ol, Il = 8192, 11008, 4096
        if a.python_rule:
            # the reference's own rule for 8192 tokens (one block of 8192, 2080 rows kept, listed run by
            # run as the layer lists them): the two-level token-wise path, which has no per-kernel pass
            from hot_amd.hadamard_matmul import run_major
            pn, prow = hla_rows(Ll)
            prow = run_major(prow)
        else:
            pn, prow = paper_rows(16, 8)
        lopt = ops.HotOptions(n_o=16, hla_n=int(pn), hla_rows=tuple(int(v) for v in prow))
        lw, lsets = make_layer(Ll, Ol, Il, torch.bfloat16, dev, nsets=2, seed=1)
        lsec, lbufs, lws = step_time(lw, lsets, lopt, a.steps, a.warmup)
        ltable = None if a.python_rule else kernel_table(lw, lsets, lbufs, lopt, lws, iters=6, warm=2)
        print(json.dumps({"workload": "Llama-7B gate/up linear backward (L=8192, O=11008, I=4096), bf16, HLA n=%d r=%d"
                                      % (lopt.hla_n, lopt.hla_r),
                          "us_per_layer": round(lsec * 1e6, 1), "steps": a.steps, "warmup": a.warmup,
                          "kernels_serial": ltable}))
        return

    L, O, I = 12608, 3072, 768
    n, rows = hla_rows(L)
    opt = ops.HotOptions(n_o=16, hla_n=int(n), hla_rows=tuple(int(v) for v in rows))
    w, sets = make_layer(L, O, I, torch.bfloat16, dev, nsets=4)
    sec, bufs, ws = step_time(w, sets, opt, a.steps, a.warmup)

    out = {
        "metric": "hot_linear_backward_us_per_layer", "value": round(sec * 1e6, 2), "unit": "us/layer",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(sec * 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "ViT-B fc1 linear backward, batch 64 x 197 tokens (L=12608, O=3072, I=768), bf16 g_y/W/out; "
                               "HQ INT4 g_x (Hadamard 16 along O) + HLA n=64 r=36 INT8 g_W; round-to-nearest, "
                               "per-tensor steps; INT8 activation buffer written beforehand",
                   "L": L, "O": O, "I": I, "input_sets_rotated": len(sets)},
    }
    if not a.no_extras:
        traffic, traffic_commit = profiled_traffic()
        table = kernel_table(w, sets, bufs, opt, ws, iters=20, warm=4, traffic=traffic)
        out["kernels"] = table
        out["traffic_source"] = ("profiles/hot_linear_backward_vit_b_fc1_bf16.hbm_traffic.txt, rocprofv3 FETCH_SIZE / WRITE_SIZE "
                                 "at commit %s" % traffic_commit) if traffic else None
        try:
            copy_gbs, mfma_tops = ops.measure_ceilings(dev)
            out["ceilings"] = {"copy_kernel_GBps": round(copy_gbs), "copy_frac_of_8TBps": round(copy_gbs / HBM_PEAK_GBS, 3),
                               "mfma_int8_loop_TOPs": round(mfma_tops), "mfma_frac_of_5POPs": round(mfma_tops / INT8_PEAK_TOPS, 3),
                               "note": "plain kernels of the library on this box: 512 MiB device copy (bytes read + written), "
                                       "loop of independent v_mfma_i32_32x32x32_i8, one wave per SIMD"}
        except Exception as e:
            out["ceilings"] = {"error": repr(e)[:200]}
        # Roofline entry: the single launch with the longest duration inside the step, measured with
        # HIP events on the launch stream around every kernel group, the groups launched one after
        # the other (the timed steps above overlap independent kernels on two streams, which
        # stretches each of them; a kernel's own duration is the serial one).  A group of two
        # launches, the split-K GEMM and its reduce kernel, is not one kernel and stands in the
        # table only.  The same two GEMMs launched back to back, without the neighbouring
        # kernels, are reported beside it.
        rows = {r["key"]: r for r in table}
        key = max((k for k in rows if rows[k]["launches"] == 1), key=lambda k: rows[k]["us"])
        dom = rows[key]
        def entry(r):
            return {"kernel": r["kernel"], "bound": r["bound"], "achieved": r["achieved"], "peak": r["peak"],
                    "unit": r["unit"], "frac": r["frac"], "traffic": r["traffic"], "us_per_launch": r["us"],
                    "per_launch": r["work"]}
        out["roofline"] = entry(dom)
        # At this workload the g_x GEMM and the token-wise quantise pass of g_y take the same time to
        # within a microsecond, and either may come out on top of a run: the longest launch of each
        # bound class is reported as well.
        out["roofline_by_bound"] = {
            b: entry(max((r for r in table if r["bound"] == b and r["launches"] == 1), key=lambda r: r["us"]))
            for b in ("mfma", "hbm")}
        if not a.table_only:
            us_gx, us_gw = gemm_launch_times(w, sets, bufs, opt)
            out["roofline"]["back_to_back_us"] = {"gemm_gx": round(us_gx, 2), "gemm_gw": round(us_gw, 2)}
    if not a.no_extras and not a.table_only:
        # Llama-7B gate/up at 8192 tokens, bf16, paper HLA setting (n = 16, 8 lowest sequencies)
        Ll, Ol, Il = 8192, 11008, 4096
        pn, prow = paper_rows(16, 8)
        lopt = ops.HotOptions(n_o=16, hla_n=int(pn), hla_rows=tuple(int(v) for v in prow))
        lw, lsets = make_layer(Ll, Ol, Il, torch.bfloat16, dev, nsets=2, seed=1)
        lsec, lbufs, lws = step_time(lw, lsets, lopt, max(5, a.steps // 5), max(2, a.warmup // 5))
        ltraffic, ltraffic_commit = profiled_traffic("llama_gate_up")
        ltable = kernel_table(lw, lsets, lbufs, lopt, lws, iters=6, warm=2, traffic=ltraffic)
        out["llama_gate_up"] = {"us_per_layer": round(lsec * 1e6, 1), "L": Ll, "O": Ol, "I": Il,
                                "hla": "n=16 r=8", "int8_tops": round((2.0 * Ll * Ol * Il + 2.0 * Ol * Il * (Ll // 2)) / lsec / 1e12, 1),
                                # kernels launched one after the other: [us, fraction of the 8 TB/s or 5 POP/s
                                # peak, HBM bytes per launch from the committed counter summary or null]
                                "kernels_serial": {r["key"]: [r["us"], r["frac"], r["traffic"]] for r in ltable},
                                "traffic_source": ("profiles/hot_linear_backward_llama_gate_up_bf16.hbm_traffic.txt at commit %s"
                                                   % ltraffic_commit) if ltraffic else None}
        # the same layer at the reference's own low-rank rule for 8192 tokens (utils/hadamard_matmul.py:209-226:
        # one block of n = 8192, r = 2080 kept sequencies; the two-level token-wise path), the kept rows
        # listed run by run as the layer lists them (hot_amd.quant_matmul.token_rule)
        try:
            from hot_amd.hadamard_matmul import run_major
            rn, rrow = hla_rows(Ll)
            rrow = run_major(rrow)
            ropt = ops.HotOptions(n_o=16, hla_n=int(rn), hla_rows=tuple(int(v) for v in rrow))
            del lbufs, lws
            rsec, rbufs, rws = step_time(lw, lsets, ropt, max(5, a.steps // 5), max(2, a.warmup // 5))
            out["llama_gate_up_python_rule"] = {"us_per_layer": round(rsec * 1e6, 1), "L": Ll, "O": Ol, "I": Il,
                                                "hla": "n=%d r=%d" % (ropt.hla_n, ropt.hla_r),
                                                "ratio_to_paper_rule": round(rsec / lsec, 3)}
            del rbufs, rws
        except Exception as e:              # an extra: never costs the headline line
            out["llama_gate_up_python_rule"] = {"error": repr(e)[:200]}
        del lw, lsets
    if not a.no_extras and not a.table_only:
        for key, fn in (("layers", lambda: layer_table(dev)), ("measure_py", lambda: measure_py(dev)),
                        ("forward_gemm", lambda: forward_gemm_table(dev)), ("schemes", lambda: scheme_table(dev)), ("host_cost", lambda: host_cost(dev))):
            try:
                out[key] = fn()
            except Exception as e:          # extras never cost the headline line
                out[key] = {"error": repr(e)[:200]}
        try:
            out["hq_rowwise_sweep"] = hq_rowwise_sweep(dev)
        except Exception as e:
            out["hq_rowwise_sweep"] = {"error": repr(e)[:200]}
        try:
            out["quantiser_grid"] = quantiser_grid(w, sets)
        except Exception as e:
            out["quantiser_grid"] = {"error": repr(e)[:200]}
        try:
            out["vit_b16"] = vit_b16_backward(dev)
        except Exception as e:          # an extra: never costs the headline line
            out["vit_b16"] = {"error": repr(e)[:200]}
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()

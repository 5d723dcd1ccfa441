#!/usr/bin/env python3
"""Headline benchmark (the default, `--config 3`): the w3 MoE layer at the speculative-verify batch (BASELINE config 3: 32 tokens, hidden 2048,
512 experts of intermediate 512 + 1 shared expert, top-10 with Zipf(1.1)-skewed routing, SiLU-gated, 3-bit weights).

A step is one MoE layer call (softmax top-k routing of given logits, expert plan, fc1, fc2, combine with the shared
expert) on one batch of 32 tokens. Steps cycle through LAYERS distinct layers (each with its own 660 MB of experts and
its own routing), so every step streams its experts from HBM, not from the 256 MB Infinity Cache. The K timed steps
are one HIP-graph replay (the way a serving engine issues them), bracketed by synchronizations.

Prints one JSON line: tokens/s (the median of repeated replays of one HIP graph of all steps, with their minimum and
maximum), the HBM roofline of the dominant kernel (the weight stream: fc1 and fc2 in one launch) measured live with HIP
events, against the vendor peak and against a plain streaming read measured in the same run, the same layer at one token
(config 2) as a sub-record `m1`, and the CPU oracle timed on this host's cores on a bounded sample of the same workload
(whole calls, and the same without the time spent unpacking weights).

The other BASELINE configs are `--config 2` (the same layer at M = 1), `--config 0` / `--config 1` (the w3 / NVFP4 dense
decode projection, `--rows` for M) and `--config 4` (the NVFP4 latent-MoE layer on a 2048-token prefill chunk, MFMA
roofline); they print the same kind of line (configs 0, 2 and 4 with a CPU leg of their own). The default run carries
configs 0, 1 and 4 as `other_configs` and config 2 as `m1`.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
M, HIDDEN, INTER, EXPERTS, TOPK, ZIPF = 32, 2048, 512, 512, 10, 1.1


def w3_bytes(n: int, k: int) -> int:
    """Bytes of a W3 matrix in the reference layout: 3 bits a weight, an E4M3 scale per 32, an FP32 row scale."""
    return n * k * 3 // 8 + n * k // 32 + 4 * n


FC1_BYTES, FC2_BYTES = w3_bytes(2 * INTER, HIDDEN), w3_bytes(HIDDEN, INTER)
EXPERT_BYTES = FC1_BYTES + FC2_BYTES  # 1 290 240


class Hip:
    """The few runtime calls the live kernel timing needs (events on the stream the kernels are launched on)."""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")

    def events(self, n):
        out = (C.c_void_p * n)()
        for i in range(n):
            ev = C.c_void_p()
            assert self.rt.hipEventCreate(C.byref(ev)) == 0
            out[i] = ev
        return out

    def elapsed_ms(self, a, b) -> float:
        ms = C.c_float()
        assert self.rt.hipEventSynchronize(C.c_void_p(b)) == 0
        assert self.rt.hipEventElapsedTime(C.byref(ms), C.c_void_p(a), C.c_void_p(b)) == 0
        return ms.value


def cpu_baseline(layer, x, ids, weights, budget_s: float = 15.0):
    """The CPU oracle's layer (oracle/c/w3_oracle.c: unpack the experts a call names from the checkpoint layout, FP32
    matmuls, SiLU gate, combine, shared expert; OpenMP over rows) on this host's cores: whole 32-token layer calls,
    repeated until about `budget_s` of CPU time is spent."""
    import numpy as np
    import torch

    from oracle import c_port

    experts, shared = layer

    def host(ex):
        u32 = lambda t: t.view(torch.int32).cpu().numpy().view(np.uint32)  # noqa: E731
        (n1, h), (_, i) = ex.shape13, ex.shape2
        return c_port.HostExperts(u32(ex.planes13), ex.scales13.cpu().numpy(), ex.row13.cpu().numpy(), u32(ex.planes2), ex.scales2.cpu().numpy(),
                                  ex.row2.cpu().numpy(), ex.codebook, ex.fc2_codebook, h, i, n1 == 2 * i)

    routed, sh = host(experts), host(shared)
    xb = x.view(torch.int16).cpu().numpy().view(np.uint16)
    idn, wn = ids.cpu().numpy(), weights.cpu().numpy()
    out, distinct = c_port.moe_layer(routed, xb, idn, wn, sh)  # warm-up, and the result the GPU is compared with below
    calls, spent, unpacking = 0, 0.0, 0.0
    while spent < budget_s and calls < 50:
        t0 = time.perf_counter()
        c_port.moe_layer(routed, xb, idn, wn, sh)
        spent += time.perf_counter() - t0
        unpacking += c_port.last_unpack_seconds()
        calls += 1
    info = {"value": x.shape[0] * calls / spent, "unit": "tokens/s", "cores": c_port.threads(), "kind": "port",
            "matmul_only": {"value": x.shape[0] * calls / max(spent - unpacking, 1e-9), "unit": "tokens/s",
                            "what": "the same calls without the time spent unpacking weights (weights as if pre-dequantized)"},
            "unpack_share": unpacking / spent,
            "sample": f"{calls} whole layer calls of {x.shape[0]} tokens on layer 0 ({distinct} distinct experts + shared): C/OpenMP oracle, "
                      f"unpack from the checkpoint layout + FP32 matmul"}
    return info, torch.from_numpy(out.view(np.int16).copy()).view(torch.bfloat16)


MFMA_BF16_PEAK_TFLOPS = 2500.0


def latent_prefill(args) -> dict:
    """BASELINE config 4 (not the headline line; `--config 4`): the NVFP4 latent-MoE layer on a prefill chunk of 2048
    tokens - hidden 4096 projected to latent 1024, 512 ReLU^2 experts of intermediate 2688, top-22 by sigmoid scores.
    A step is the whole block (fused router|fc1_latent GEMM, routing, plan, the two expert GEMMs on the MFMA tile kernel,
    combine, fc2_latent GEMM); the roofline entry is the fc1 expert GEMM against the dense BF16 MFMA peak."""
    import torch

    from hibana_amd import _lib, synthetic
    from hibana_amd.model import nemotron_moe

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    tokens, hidden, latent, inter, experts, topk = 2048, 4096, 1024, 2688, 512, 22
    g = torch.Generator(device=dev).manual_seed(5)
    ex = synthetic.nvfp4_experts(experts, latent, inter, 11, dev, keep=not args.no_cpu)
    router = torch.randn(experts, hidden, device=dev, generator=g) * (1.0 / hidden ** 0.5)  # logits ~ N(0, 1) for x ~ N(0, 1)
    fc1 = torch.randn(latent, hidden, device=dev, generator=g) * 0.02
    fc2 = (torch.randn(hidden, latent, device=dev, generator=g) * 0.02).bfloat16()
    block = nemotron_moe.NemotronMoe(torch.cat([router, fc1]).bfloat16(), torch.zeros(experts, device=dev), fc2, ex, topk)
    x = torch.randn(tokens, hidden, device=dev, generator=g).bfloat16()
    for _ in range(max(args.warmup, 2)):
        block(x)
    torch.cuda.synchronize()
    hip = Hip()
    names = ["route", "plan count", "plan scan", "plan place", "fc1", "fc2", "combine"]  # 45 056 pairs: the plan is three launches
    per_kernel = {n: [] for n in names}
    for rep in range(4):
        evs = hip.events(2 * len(names))
        _lib.check(_lib.lib().hb_debug_events(evs, len(evs)), "events")
        block(x)
        _lib.lib().hb_debug_events(None, 0)
        torch.cuda.synchronize()
        if rep:
            for j, n in enumerate(names):
                per_kernel[n].append(hip.elapsed_ms(evs[2 * j], evs[2 * j + 1]))
    mean = lambda v: sum(v) / len(v)  # noqa: E731
    steps = max(1, args.steps // 10)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = [block(x) for _ in range(steps)]
    times = replay_times(graph, steps)
    elapsed = median(times) * 1e-3 * steps
    del outs
    gemm_flops = tokens * topk * 2 * inter * latent  # one expert GEMM (fc1 or fc2), useful flops
    fc1_ms = mean(per_kernel["fc1"])
    mfma_tflops = mfma_rate_tflops(dev)
    cpu, check = None, None
    if not args.no_cpu:
        cpu, check = latent_cpu_leg(block, ex, fc1.bfloat16().cpu(), fc2.cpu(), x, latent, inter)
    small = latent_small_calls(block, ex, hidden, dev, g)
    line = {
        "metric": "NVFP4 latent-MoE layer tokens/s on a 2048-token prefill chunk, with achieved MFMA TFLOP/s",
        "value": tokens * steps / elapsed, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": elapsed / steps * 1e3, "ms_per_step_min": times[0], "ms_per_step_max": times[-1], "replays": len(times),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 4: NVFP4 latent-MoE layer, 2048 tokens, hidden 4096 -> latent 1024, 512 experts x inter 2688, "
                               "ReLU^2, top-22 sigmoid routing of N(0,1) logits, no shared expert",
                   "timed_as": "replays of one HIP graph of all steps; value and ms_per_step are the median replay"},
        "roofline": {"bound": "mfma", "kernel": "tile_kernel<TileNvfp4, fc1 relu2>", "achieved": gemm_flops / (fc1_ms * 1e-3) / 1e12,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": gemm_flops / (fc1_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": None, "launch_flops": gemm_flops, "launch_ms": fc1_ms, "peak_measured": mfma_tflops,
                     "frac_of_measured": gemm_flops / (fc1_ms * 1e-3) / 1e12 / mfma_tflops,
                     "peak_measured_how": "BF16 16x16x32 MFMAs on registers alone in this run (hb_debug_mfma_rate)"},
        "layer_chain": {"kernel_ms": {n: mean(v) for n, v in per_kernel.items()}},
        "decode_calls": small,
        "cpu_baseline": cpu,
        "parity": check,
    }
    return line


def latent_small_only(args) -> dict:
    """`--config 4 --small-rows M`: config 4's block with the shared expert at M rows through the small-call kernels
    alone (a profiling mode: its kernel trace shows the six launches of a decode or verify call)."""
    import torch

    from hibana_amd import synthetic
    from hibana_amd.model import nemotron_moe

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    hidden, latent, inter, experts, topk, shared_inter, m = 4096, 1024, 2688, 512, 22, 5376, args.small_rows
    g = torch.Generator(device=dev).manual_seed(5)
    ex = synthetic.nvfp4_experts(experts, latent, inter, 11, dev)
    gate_fc1 = torch.cat([torch.randn(experts, hidden, device=dev, generator=g) * (1.0 / hidden ** 0.5), torch.randn(latent, hidden, device=dev, generator=g) * 0.02])
    fc2 = (torch.randn(hidden, latent, device=dev, generator=g) * 0.02).bfloat16()
    block = nemotron_moe.NemotronMoe(gate_fc1.bfloat16(), torch.zeros(experts, device=dev), fc2, ex, topk, synthetic.nvfp4_linear(shared_inter, hidden, 61, dev),
                                     synthetic.nvfp4_linear(hidden, shared_inter, 62, dev))
    xs = [torch.randn(m, hidden, device=dev, generator=g).bfloat16() for _ in range(8)]
    for x in xs:
        block.small(x)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = [block.small(xs[i % 8]) for i in range(args.steps)]
    times = replay_times(graph, args.steps)
    del outs
    return {"metric": "NVFP4 latent-MoE block microseconds a call through the small-call kernels", "rows": m, "us_per_call": median(times) * 1e3,
            "us_per_call_min": times[0] * 1e3, "us_per_call_max": times[-1] * 1e3, "steps": args.steps, "replays": len(times)}


def latent_small_calls(block, ex, hidden: int, dev, g, shared_inter: int = 5376):
    """The same block with a shared expert of intermediate 5376 at 1, 4 and 16 rows (decode and verify calls):
    microseconds a call through the small-call kernels (router, block: six launches) and through the operators a
    longer call uses (two GEMMs, routing, plan, two expert layers, combine, the shared expert's two linears: nine), each
    as replays of a graph of 32 calls over 8 inputs."""
    import torch

    from hibana_amd import synthetic
    from hibana_amd.model import nemotron_moe

    up, down = synthetic.nvfp4_linear(shared_inter, hidden, 61, dev), synthetic.nvfp4_linear(hidden, shared_inter, 62, dev)
    both = nemotron_moe.NemotronMoe(block.gate_fc1, block.bias, block.fc2, ex, block.topk, up, down)

    def operators(x):
        fused = torch.mm(x, both.gate_fc1.T, out_dtype=torch.float32)
        ids, w, lat = both.route(fused)
        return torch.addmm(both.shared(x), both.routed(lat, ids, w), both.fc2.T)

    out = {"workload": f"config 4's block with a shared expert of intermediate {shared_inter}, M = 1 / 4 / 16 rows of N(0,1)"}
    for m in (1, 4, 16):
        xs = [torch.randn(m, hidden, device=dev, generator=g).bfloat16() for _ in range(8)]
        row = {}
        for name, fn in (("small_call_kernels_us", both.small), ("operators_us", operators)):
            for x in xs:
                fn(x)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                outs = [fn(x) for x in xs for _ in range(4)]
            row[name] = median(replay_times(graph, 32)) * 1e3
            del outs, graph
        out[str(m)] = row
    return out


def latent_cpu_leg(block, ex, fc1, fc2, x, latent: int, inter: int, rows: int = 12):
    """The CPU oracle of the latent-MoE block (oracle/layers.py: per distinct expert, unpack the NVFP4 matrices, BF16
    linears with FP32 accumulation, ReLU^2, weighted FP32 sum, then the latent projection back) on a seeded sample of
    `rows` token rows - a row's output depends on its own experts only - timed on this host's cores, and the GPU's rows
    against it."""
    import numpy as np
    import torch

    from oracle import layers, nvfp4_format as onv
    dev = x.device
    sample = torch.randperm(x.shape[0], generator=torch.Generator().manual_seed(1))[:rows].sort().values
    fused = torch.mm(x, block.gate_fc1.T, out_dtype=torch.float32)
    ids, w, _ = block.route(fused)
    got = block(x)[sample.to(dev)].cpu()
    host = {}  # the experts the sample names, as the checkpoint holds them, copied before the clock starts
    for i in torch.unique(ids[sample.to(dev)]).tolist():
        host[i] = (ex.w1[i].cpu().numpy(), ex.s1[i].view(torch.uint8).cpu().numpy(), float(ex.alpha1[i]), ex.w2[i].cpu().numpy(),
                   ex.s2[i].view(torch.uint8).cpu().numpy(), float(ex.alpha2[i]))

    def get(i):
        w1, s1, a1, w2, s2, a2 = host[i]
        return (onv.unpack_fp4(w1, onv.unswizzle_block_scales(s1, inter, latent // 16)), np.float32(a1),
                onv.unpack_fp4(w2, onv.unswizzle_block_scales(s2, latent, inter // 16)), np.float32(a2))

    xs, ids_s, w_s = x[sample.to(dev)].cpu(), ids[sample.to(dev)].cpu().numpy(), w[sample.to(dev)].cpu()
    t0 = time.perf_counter()
    want = layers.latent_moe_ref(xs, fc1, fc2, ids_s, w_s, get)
    spent = time.perf_counter() - t0
    cpu = {"value": rows / spent, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
           "sample": f"{rows} seeded token rows of the 2048 ({len(host)} distinct experts): numpy / torch oracle, unpack from the checkpoint layout + "
                     f"matmuls, one call of {spent:.1f} s"}
    a, e = got.double(), want.double()
    check = {"rows_checked": rows, "max_rel_vs_cpu_oracle": float((a - e).abs().max() / e.abs().max()), "norm_rel_vs_cpu_oracle": float((a - e).norm() / e.norm())}
    return cpu, check


def dense_decode(args) -> dict:
    """BASELINE configs 0 and 1 (not the headline line): one dense decode projection a step - config 0 the w3 linear
    5120 x 5120 at M = 1, config 1 the NVFP4 up-projection 25600 x 5120 at M = --rows (1, 8 or 64) - cycling through six
    copies of the matrix so that every step streams its weights from HBM. The roofline entry is that one kernel against
    the HBM peak, its duration from the kernel's own start / stop events."""
    import torch

    from hibana_amd import _lib, synthetic
    from hibana_amd.kernels import w3

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.lib()
    m = args.rows
    if args.config == 0:
        n = k = 5120
        nbytes = w3_bytes(n, k)
        args.layers = max(args.layers, -(-320_000_000 // nbytes))  # more than the 256 MB Infinity Cache holds, so that every step streams from HBM
        book = args.codebook  # "lloyd2": a two-bit matrix, streamed at 2.25 bits a weight
        bits = 2 if book == "lloyd2" else 3
        nbytes = n * k * bits // 8 + n * k // 32 + 4 * n
        mats = [w3.tile(synthetic.w3_matrix(n, k, 40 + i, dev, book), release=bool(i) or args.no_cpu) for i in range(args.layers)]  # the CPU leg reads matrix 0 in the checkpoint layout
        x = torch.randn(m, k, generator=torch.Generator().manual_seed(3)).bfloat16().to(dev)

        def step(i: int):
            return w3.w3_linear(x, mats[i % args.layers])

        kernel, what = "w3_stream_kernel<dense>", f"BASELINE config 0: w3 dense linear {n} x {k}, M = {m}, {book} codebook" + (" (two-bit tiles)" if bits == 2 else "")
    else:
        n, k = 25600, 5120
        size = lib.hb_nvfp4_tiled_bytes(n, k)
        g = torch.Generator(device=dev).manual_seed(7)
        mats = [torch.randint(0, 256, (size,), dtype=torch.uint8, device=dev, generator=g) for _ in range(args.layers)]
        for t in mats:  # every scale byte a finite positive E4M3 value
            blocks = t.view(-1, 4608)[:, 4096:]
            blocks.copy_(blocks % 120 + 1)
        nbytes = n * k // 2 + n * k // 16

        def call(rows: int):
            """(step, kernel name) of the projection at `rows` activation rows, its workspace (the partial tiles of a
            call whose tiles share K among workgroups) allocated once."""
            xr = torch.randn(rows, k, generator=torch.Generator().manual_seed(3)).bfloat16().to(dev)
            yr = torch.empty(rows, n, dtype=torch.bfloat16, device=dev)
            need = lib.hb_nvfp4_gemm_workspace_bytes(rows, n, k)
            ws = torch.zeros(max(need, 16), dtype=torch.uint8, device=dev)  # a workspace starts with its head zero

            def run(i: int):
                _lib.check(lib.hb_nvfp4_gemm_ws(_lib.ptr(xr), rows, _lib.ptr(mats[i % args.layers]), 1.0 / 448.0, n, k, 0, _lib.ptr(yr), _lib.ptr(ws), need,
                                                _lib.stream()), "nvfp4 gemm")
                return yr

            return run, "tile_kernel<TileNvfp4, dense>, K shared among workgroups" if need else "nvfp4_stream_kernel<dense>"

        step, kernel = call(m)
        what = f"BASELINE config 1: NVFP4 dense linear {n} x {k}, M = {m} (codes and block scales random, global scale 1/448)"
    for i in range(max(args.warmup, args.layers)):
        step(i)
    torch.cuda.synchronize()
    hip = Hip()
    times = []
    for rep in range(5):
        for i in range(args.layers):
            evs = hip.events(2)
            _lib.check(lib.hb_debug_events(evs, 2), "events")
            step(i)
            lib.hb_debug_events(None, 0)
            torch.cuda.synchronize()
            if rep:
                times.append(hip.elapsed_ms(evs[0], evs[1]))
    kernel_ms = sum(times) / len(times)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = [step(i) for i in range(args.steps)]
    times = replay_times(graph, args.steps)
    elapsed = median(times) * 1e-3 * args.steps
    del outs
    achieved = nbytes / (kernel_ms * 1e-3) / 1e9
    if args.copy_mib:  # a plain device copy of known size, for scaling the counters of a rocprofv3 --pmc run
        src = torch.empty(args.copy_mib << 20, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    ratio = traffic_ratio(f"traffic_ratio_config{args.config}_m1", "decode_configs_0_1_hbm_traffic.md") if m == 1 else None
    by_rows = None
    if args.config == 1:  # the same projection at the configuration's other row counts: microseconds a call, graph-replayed
        by_rows = {}
        for rows in (1, 8, 64):
            run, name = call(rows)
            for i in range(args.layers):
                run(i)
            torch.cuda.synchronize()
            g2 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g2):
                outs = [run(i) for i in range(args.steps)]
            by_rows[str(rows)] = {"us_per_call": median(replay_times(g2, args.steps)) * 1e3, "kernel": name}
            del outs, g2
    cpu, check = None, None
    if args.config == 0 and not args.no_cpu:
        # BASELINE config 0 is the reference's own CPU-runnable case: the C oracle's dense product (unpack the matrix from
        # the checkpoint layout, FP32 matmul; OpenMP over the output rows) on this host's cores, whole calls for a few seconds
        import numpy as np

        from oracle import c_port
        w0 = mats[0]
        host = {"planes": w0.planes.view(torch.int32).cpu().numpy().view(np.uint32), "scales": w0.scales.cpu().numpy(), "row_scale": w0.row_scale.cpu().numpy(),
                "out_features": n, "in_features": k, "codebook": w0.codebook}
        xb = x.view(torch.int16).cpu().numpy().view(np.uint16)
        want = c_port.linear(host, xb)
        calls, spent = 0, 0.0
        while spent < 8.0 and calls < 200:
            t0 = time.perf_counter()
            c_port.linear(host, xb)
            spent += time.perf_counter() - t0
            calls += 1
        cpu = {"value": m * calls / spent, "unit": "tokens/s", "cores": c_port.threads(), "kind": "port",
               "sample": f"{calls} whole calls of the {n} x {k} product at M = {m} on matrix 0: C/OpenMP oracle, unpack from the checkpoint layout + FP32 matmul"}
        got = step(0).float().cpu()
        ref = torch.from_numpy(want.view(np.int16).copy()).view(torch.bfloat16).float()
        check = {"max_rel_vs_cpu_oracle": float((got - ref).abs().max() / ref.abs().max()), "norm_rel_vs_cpu_oracle": float((got - ref).norm() / ref.norm())}
    line = {
        "metric": "dense decode projection tokens/s, with achieved HBM GB/s", "value": m * args.steps / elapsed, "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": elapsed / args.steps * 1e3, "ms_per_step_min": times[0], "ms_per_step_max": times[-1],
        "replays": len(times), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": what, "matrices_cycled": args.layers, "timed_as": "replays of one HIP graph of all steps; median replay"},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     # HBM bytes a launch: scaled FETCH_SIZE + WRITE_SIZE over the algorithmic bytes, measured with
                     # rocprofv3 --pmc on this workload (the summary under profiles/ states it), applied to this run's bytes
                     "traffic": None if ratio is None else ratio * nbytes, "launch_bytes": nbytes, "launch_ms": kernel_ms},
        "cpu_baseline": cpu,
        "parity": check,
    }
    if by_rows:
        line["by_rows"] = by_rows
    return line


def routing_only(args) -> dict:
    """`--routing [ROWS]`: the routing launches alone at Flash-Next's router shape (512 experts, top 10), graph-replayed:
    `route_topk` and the budgeted `route_budget` (keep 4, budget 64) at decode / verify row counts."""
    import torch

    from hibana_amd.kernels import ops

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    g = torch.Generator(device=dev).manual_seed(7)
    rows_out = {}
    for rows in ((args.routing,) if args.routing else (1, 16, 64, 320)):
        feeds = [(torch.randn(rows, 512, device=dev, generator=g) * 1.2).bfloat16() for _ in range(8)]
        floats = [f.float() for f in feeds]
        entry = {}
        for name, call in (("route_topk", lambda i: ops.route_topk(floats[i % 8], 10)), ("route_budget", lambda i: ops.route_budget(feeds[i % 8], 10, 4, 64))):
            call(0)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                outs = [call(i) for i in range(args.steps)]
            entry[name + "_us"] = round(median(replay_times(graph, args.steps)) * 1e3, 2)
            del outs, graph
        rows_out[str(rows)] = entry
    return {"metric": "routing microseconds a call (512 experts, top 10; budgeted: keep 4, budget 64)", "by_rows": rows_out, "steps": args.steps}


def replay_times(graph, steps: int, floor_s: float = 0.2, least: int = 5):
    """Per-step milliseconds of repeated replays of a graph of `steps` steps: at least `least` replays and at least
    `floor_s` seconds of them, each bracketed by synchronizations."""
    import torch
    graph.replay()  # untimed: the first replay uploads the graph
    torch.cuda.synchronize()
    out, total = [], 0.0
    while len(out) < least or total < floor_s:
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        out.append(dt / steps * 1e3)
        total += dt
    return sorted(out)


def median(values):
    v = sorted(values)
    return v[len(v) // 2] if len(v) % 2 else 0.5 * (v[len(v) // 2 - 1] + v[len(v) // 2])


def stream_read_gbs(dev, mib: int = 1024) -> float:
    """What a kernel that only reads gets from this device's memory: a plain 128-bit-load streaming read of `mib` MiB
    (hb_debug_stream_read), median of seven runs timed with events on the stream it runs on."""
    import torch

    from hibana_amd import _lib
    src = torch.empty(mib << 20, dtype=torch.uint8, device=dev).random_()
    sink = torch.zeros((mib << 20) // 65536 + 1, dtype=torch.int32, device=dev)
    times = []
    for i in range(9):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _lib.check(_lib.lib().hb_debug_stream_read(_lib.ptr(src), src.numel(), _lib.ptr(sink), _lib.stream()), "stream read")
        e1.record()
        torch.cuda.synchronize()
        if i >= 2:
            times.append(e0.elapsed_time(e1))
    return src.numel() / (median(times) * 1e-3) / 1e9


def ring_skeleton_gbs(dev, experts: int = 137, regions: int = 6) -> float:
    """What the W3 stream's request structure gets without its arithmetic (hb_debug_ring_skeleton): `experts` x 16
    blocks of 53 248 bytes - fc1 of a verify step - at expert-sized runs scattered over a region four times as large,
    four wavefronts a block, each four chunks through the two-slot LDS ring, activations beside them, the K split's
    exchange and a store; a region a launch out of `regions` (nothing stays in the caches); twelve launches one after the
    other between two events, the median repetition's time a launch."""
    import torch

    from hibana_amd import _lib
    place_bytes, groups = 53248, experts * 16
    region = 4 * groups * place_bytes
    src = torch.empty(regions * region, dtype=torch.uint8, device=dev).random_()
    order = torch.randperm(4 * experts, generator=torch.Generator().manual_seed(7))[:experts]
    table = (order[:, None] * 16 + torch.arange(16)[None, :]).reshape(-1).to(torch.int32).to(dev)
    acts = torch.zeros(32 * 4096, dtype=torch.uint8, device=dev)
    out = torch.empty(groups * 256, dtype=torch.float32, device=dev)
    sink = torch.zeros(groups, dtype=torch.int32, device=dev)
    def launch(i: int):
        at = src[(i % regions) * region:(i % regions + 1) * region]
        _lib.check(_lib.lib().hb_debug_ring_skeleton(_lib.ptr(at), at.numel(), _lib.ptr(table), groups, _lib.ptr(acts), acts.numel(), _lib.ptr(out),
                                                     out.numel() * 4, _lib.ptr(sink), sink.numel() * 4, _lib.stream()), "ring skeleton")

    times = []
    for rep in range(6):  # the launches of a repetition follow one another on the stream, as a graph's kernels do
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(2 * regions):
            launch(i)
        e1.record()
        torch.cuda.synchronize()
        if rep:
            times.append(e0.elapsed_time(e1) / (2 * regions))
    return groups * place_bytes / (median(times) * 1e-3) / 1e9


def mfma_rate_tflops(dev, blocks: int = 2048, iters: int = 4096) -> float:
    """What a kernel that only multiplies gets from this device's matrix cores: BF16 16x16x32 MFMAs on registers, eight
    wavefronts a workgroup (hb_debug_mfma_rate), median of seven runs timed with events on the stream it runs on."""
    import torch

    from hibana_amd import _lib
    sink = torch.zeros(blocks, dtype=torch.float32, device=dev)
    times, flops = [], 0
    for i in range(9):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        flops = _lib.lib().hb_debug_mfma_rate(blocks, iters, _lib.ptr(sink), _lib.stream())
        e1.record()
        torch.cuda.synchronize()
        if flops <= 0:
            raise RuntimeError(f"hb_debug_mfma_rate: {flops}")
        if i >= 2:
            times.append(e0.elapsed_time(e1))
    return flops / (median(times) * 1e-3) / 1e12


def traffic_ratio(name: str = "traffic_ratio_fc1_fc2", summary: str = "w3_moe_layer_config3_hbm_traffic.md"):
    """HBM bytes a launch / algorithmic bytes of a kernel (by default the fc1 + fc2 launch), from the committed counter
    summary (two rocprofv3 --pmc runs scaled by a plain copy of known size); None when the summary does not state it."""
    import os
    import re
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", summary)
    try:
        found = re.search(r"^" + name + r"\s*=\s*([0-9.]+)", open(path).read(), re.M)
    except OSError:
        return None
    return float(found.group(1)) if found else None


def measure_layer(args, layers, x, logits, m: int, hip, with_kernels: bool = True):
    """Replays and per-kernel times of the w3 MoE layer on `m` tokens (x, per-layer logits)."""
    import torch

    from hibana_amd import _lib
    from hibana_amd.kernels import w3_moe

    def step(i: int):
        return w3_moe.moe_layer_logits(layers[i % args.layers][0], x, logits[i % args.layers], TOPK, shared=layers[i % args.layers][1], e4m3=args.e4m3)

    for i in range(max(args.warmup, args.layers)):  # untimed: also builds every layer's tiled weights and warms the allocator
        step(i)
    torch.cuda.synchronize()
    # live kernel timing: each kernel of the chain is launched with its own (start, stop) HIP event pair, which the
    # runtime stamps with that kernel's begin and end on the stream it runs on
    if m == 1 and not args.e4m3:
        names = ["route + fc1", "fc2 + combine"]  # one token: fc1's wavefronts route the row themselves; fc2 and the combine are one launch
    elif m == 1:
        names = ["route + plan", "fc1", "fc2 + combine"]  # up to 4 rows are routed by the plan's workgroup
    elif args.e4m3:
        names = ["route + plan", "fc1", "fc2", "combine"]
    else:
        names = ["route + plan", "fc1 + fc2", "combine"]  # the last routing workgroup plans; fc2's workgroups wait for their slot's fc1 inside one launch
    per_kernel = {n: [] for n in names}
    for rep in range(5):
        for i in range(args.layers):
            evs = hip.events(2 * len(names))
            for lead in range(3):  # the timed step runs behind three others on a busy stream, as a graph's steps do
                step(i + 1 + lead)
            _lib.check(_lib.lib().hb_debug_events(evs, len(evs)), "events")
            step(i)
            _lib.lib().hb_debug_events(None, 0)
            torch.cuda.synchronize()
            ms = [hip.elapsed_ms(evs[2 * j], evs[2 * j + 1]) for j in range(len(names))]
            if rep:  # the first sweep is untimed
                for n, v in zip(names, ms):
                    per_kernel[n].append(v)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = [step(i) for i in range(args.steps)]
    times = replay_times(graph, args.steps)
    del outs, graph
    return times, {n: sum(v) / len(v) for n, v in per_kernel.items()}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=24)
    ap.add_argument("--layers", type=int, default=6, help="distinct layers the steps cycle through")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--config", type=int, default=3, choices=(0, 1, 2, 3, 4),
                    help="3: the headline w3 verify-batch layer (with the M = 1 layer as a sub-record); 2: the same layer at M = 1 alone; 0 / 1: the "
                         "w3 / NVFP4 dense decode projection; 4: the NVFP4 prefill layer")
    ap.add_argument("--rows", type=int, default=1, help="configs 0 and 1: activation rows M")
    ap.add_argument("--codebook", default="uniform", choices=("uniform", "lloyd", "zero8", "lloyd2"),
                    help="config 0: the matrix's codebook (lloyd2: four levels, the two-bit tile layout)")
    ap.add_argument("--small-rows", type=int, default=0, help="config 4: only its block (with a shared expert) at this many rows (1 .. 16) through the "
                    "small-call kernels")
    ap.add_argument("--routing", type=int, nargs="?", const=0, default=None, metavar="ROWS",
                    help="only the routing launches (route_topk, route_budget) at ROWS rows (none given: 1 / 16 / 64 / 320)")
    ap.add_argument("--headline-only", action="store_true", help="config 3 without the other configurations' lines (profiling runs)")
    ap.add_argument("--e4m3", action="store_true", help="configs 2 and 3: the reference kernel's own arithmetic (activations rounded to E4M3 per "
                    "32-group, FP8 MFMA) instead of the weight-only form; no CPU leg")
    ap.add_argument("--copy-mib", type=int, default=0, help="also run one plain device copy of this many MiB (a known-size "
                    "reference for scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    ap.add_argument("--tune", default="", metavar="KEY=VALUE[,KEY=VALUE]",
                    help="measurement switches of the library (hb_tune) for a profiling run; the line says so in config.tune")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no sharding, no collectives); run with --gpus 1", file=sys.stderr)
        return 2
    import torch

    from hibana_amd import synthetic
    from hibana_amd.kernels import ops, w3_moe

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels have no CPU path", file=sys.stderr)
        return 2
    tuned = {}
    for item in filter(None, args.tune.split(",")):
        from hibana_amd import _lib
        key, _, value = item.partition("=")
        _lib.check(_lib.lib().hb_tune(key.encode(), int(value)), f"hb_tune({key})")
        tuned[key] = int(value)

    def emit(line: dict) -> int:
        if tuned:
            line.setdefault("config", {})["tune"] = tuned  # not the library's built-in choices: a profiling line
        print(json.dumps(line))
        return 0

    if args.routing is not None:
        return emit(routing_only(args))
    if args.config == 4:
        return emit(latent_small_only(args) if args.small_rows else latent_prefill(args))
    if args.config in (0, 1):
        return emit(dense_decode(args))
    if args.e4m3:
        args.no_cpu = True  # the C oracle states the weight-only form
    decode = args.config == 2  # the layer at batch 1: logits from N(0, 1), ten experts and the shared one a step
    m = 1 if decode else M
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    layers = []
    for i in range(args.layers):
        keep = i == 0 and not args.no_cpu  # the CPU leg reads layer 0 in the checkpoint layout
        layers.append((synthetic.w3_experts(EXPERTS, HIDDEN, INTER, True, 100 + i, dev, release=not keep),
                       synthetic.w3_experts(1, HIDDEN, INTER, True, 900 + i, dev, release=not keep)))
    one_logits = [torch.randn(1, EXPERTS, generator=torch.Generator().manual_seed(3000 + i)).to(dev) for i in range(args.layers)]
    logits = one_logits if decode else [synthetic.zipf_logits(m, EXPERTS, ZIPF, 3000 + i, dev) for i in range(args.layers)]
    x = torch.randn(m, HIDDEN, generator=torch.Generator().manual_seed(3)).bfloat16().to(dev)
    torch.cuda.synchronize()
    hip = Hip()
    distinct = [int(torch.unique(ops.route_topk(lg, TOPK)[0]).numel()) for lg in logits]
    mean = lambda v: sum(v) / len(v)  # noqa: E731

    times, kernel_ms = measure_layer(args, layers, x, logits, m, hip)
    ms_per_step = median(times)
    step_bytes = mean([(distinct[i % args.layers] + 1) * EXPERT_BYTES + 2 * m * HIDDEN * 2 for i in range(args.steps)])
    chain_gbs = step_bytes / (ms_per_step * 1e-3) / 1e9
    # the dominant kernel: the weight stream - one launch for fc1 and fc2 (every distinct expert's and the shared expert's
    # two matrices, read once), or, at one token and in the E4M3 mode, fc1's launch
    fused = "fc1 + fc2" in kernel_ms
    routed_in_fc1 = "route + fc1" in kernel_ms  # one token: fc1's wavefronts route the row themselves
    dominant = "fc1 + fc2" if fused else "route + fc1" if routed_in_fc1 else "fc1"
    launch_bytes = mean([(d + 1) * (EXPERT_BYTES if fused else FC1_BYTES) for d in distinct])
    launch_ms = kernel_ms[dominant]
    achieved = launch_bytes / (launch_ms * 1e-3) / 1e9
    kernel_name = ("w3_fc12_kernel<fc1 gated + fc2>" if fused else "w3_fc1_route_one_kernel<route + fc1 gated>" if routed_in_fc1
                   else "w3_stream_kernel<fc1 gated, E4M3>" if args.e4m3 else "w3_stream_kernel<fc1 gated>")
    read_gbs = stream_read_gbs(dev)
    skeleton_gbs = None if decode else ring_skeleton_gbs(dev, experts=round(mean(distinct)) + 1)

    m1 = None
    if not decode:  # the other half of the metric, in the same run: the layer at one token
        x1 = x[:1].contiguous()
        d1 = [int(torch.unique(ops.route_topk(lg, TOPK)[0]).numel()) for lg in one_logits]
        t1, k1 = measure_layer(args, layers, x1, one_logits, 1, hip)
        b1 = mean([(d + 1) * EXPERT_BYTES + 2 * HIDDEN * 2 for d in d1])
        ms1 = median(t1)
        m1 = {"workload": "BASELINE config 2: the same layer at 1 token, top-10 of N(0,1) logits", "value": 1.0 / (ms1 * 1e-3), "unit": "tokens/s",
              "ms_per_step": ms1, "ms_per_step_min": t1[0], "ms_per_step_max": t1[-1], "replays": len(t1), "distinct_experts_per_step": mean(d1),
              "algorithmic_bytes_per_step": b1, "achieved_GBs": b1 / (ms1 * 1e-3) / 1e9, "frac_of_hbm_peak": b1 / (ms1 * 1e-3) / 1e9 / HBM_PEAK_GBS,
              "kernel_ms": k1}

    if args.copy_mib:
        src = torch.empty(args.copy_mib << 20, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    ids0, w0 = ops.route_topk(logits[0], TOPK)
    cpu, check = None, None
    if not args.no_cpu:
        cpu, want = cpu_baseline(layers[0], x, ids0, w0)
        got = w3_moe.moe_layer(layers[0][0], x, ids0, w0, shared=layers[0][1]).float().cpu()
        check = {"max_rel_vs_cpu_oracle": float((got - want.float()).abs().max() / want.float().abs().max()),
                 "norm_rel_vs_cpu_oracle": float((got - want.float()).norm() / want.float().norm())}
    ratio = None if decode or args.e4m3 or not fused else traffic_ratio()
    line = {
        "metric": ("w3 MoE layer tokens/s at decode (M=1), with achieved HBM GB/s" if decode else
                   "w3 MoE layer tokens/s at the verify batch (M=32), with achieved HBM GB/s") + (" [E4M3 activation mode]" if args.e4m3 else ""),
        "value": m / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_min": times[0], "ms_per_step_max": times[-1], "replays": len(times),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8" if args.e4m3 else "bf16",
        "data": "synthetic",
        "config": {"workload": ("BASELINE config 2: w3 MoE layer, 1 token, hidden 2048, 512 experts x inter 512 + 1 shared, top-10 of N(0,1) logits, "
                                "SiLU-gated, codebook lloyd") if decode else
                               ("BASELINE config 3: w3 MoE layer, 32 tokens (4 seq x 8 draft), hidden 2048, 512 experts x inter 512 + 1 shared, "
                                "top-10 Zipf(1.1) routing, SiLU-gated, codebook lloyd"),
                   "layers_cycled": args.layers, "distinct_experts_per_step": mean(distinct),
                   "timed_as": "replays of one HIP graph of all steps; value and ms_per_step are the median replay"},
        "roofline": {"bound": "hbm", "kernel": kernel_name, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     # HBM bytes a launch: the ratio of scaled FETCH_SIZE + WRITE_SIZE to the algorithmic bytes measured with
                     # rocprofv3 --pmc on this workload (the summary under profiles/ states it), applied to this run's bytes
                     "traffic": None if ratio is None else ratio * launch_bytes, "launch_bytes": launch_bytes, "launch_ms": launch_ms,
                     "peak_measured": read_gbs, "frac_of_measured": achieved / read_gbs,
                     "peak_measured_how": "plain streaming read of 1 GiB in this run (hb_debug_stream_read)",
                     # fc1's traffic of this step without the arithmetic: blocks of 53 KB at expert-sized runs, four chunks
                     # a wavefront through the two-slot LDS ring, activations beside them, the exchange and a store
                     "skeleton": skeleton_gbs, "frac_of_skeleton": None if skeleton_gbs is None else achieved / skeleton_gbs,
                     "skeleton_how": "the stream's requests without its arithmetic in this run (hb_debug_ring_skeleton)"},
        "layer_chain": {"algorithmic_bytes_per_step": step_bytes, "achieved_GBs": chain_gbs, "frac_of_hbm_peak": chain_gbs / HBM_PEAK_GBS,
                        "kernel_ms": kernel_ms},
        "m1": m1,
        "cpu_baseline": cpu,
        "parity": check,
    }
    if not decode and not args.e4m3 and not args.headline_only:
        # the other configurations' lines in the same run, each as its own mode would print it (their CPU legs kept short)
        del layers, x, logits, one_logits
        torch.cuda.empty_cache()
        others = {}
        for name, mode, overrides in (("config0", dense_decode, {"config": 0, "rows": 1}), ("config1", dense_decode, {"config": 1, "rows": 1}),
                                      ("config4", latent_prefill, {"config": 4})):
            sub = argparse.Namespace(**{**vars(args), **overrides})
            try:
                others[name] = mode(sub)
            except Exception as err:  # the headline line stands on its own
                others[name] = {"error": f"{type(err).__name__}: {err}"}
            torch.cuda.empty_cache()
        line["other_configs"] = others
    return emit(line)


if __name__ == "__main__":
    sys.exit(main())

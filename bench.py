"""Benchmark of the MoE hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu-baseline] [--skip-secondary] [--lib FILE.so]

A step is one forward+backward of the Mixtral-shape MoE layer of the baseline (T=16,384 tokens, H=4096, E=8, top-2,
I=14,336, SwiGLU, bf16 with fp32 accumulation, Zipf(1.0) expert load, synthetic data, inputs resident in HBM).
Prints ONE JSON line: whole-layer TFLOP/s (expert-GEMM FLOPs 18*R*H*I over wall time, router and bookkeeping time
included), the roofline record of the dominant kernel measured with events on the launch stream inside the timed
region, and the torch CPU path (oracle/) timed on this box's host cores on a bounded sample.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "cute-kernels_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_FP8_TFLOPS = 5000.0
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E

# Bytes per launch between L2 and the fabric (fetched + written) are not measurable from inside this process: they come
# from two rocprofv3 --pmc runs of this same command (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), summarised per
# kernel name by `bench.py --summarize-pmc` into the tracked file below. A kernel whose name is not in that file (the
# kernel changed since the counters were read) reports traffic null.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "grouped_gemm_c3_hbm_traffic.txt")


def canonical_kernel_name(name: str) -> str:
    """One spelling for the grouped GEMM kernel's instantiations, whichever way a rocprofv3 output file spells them: the
    kernel trace and the counter files of one run mix mangled names (..grouped_gemm_line_kernelIDF16bLi4ELi256ELb1ELi2ELb0EE..),
    demangled ones, and a mis-demangled form in which `DF16bLi1E` (bf16, 1) comes out as `bool _Accum, int, E`.
    -> "grouped_gemm_line_kernel<bf16, 4, 256, true, 2, false>"; other kernels keep their name."""
    import re

    m = re.search(r"grouped_gemm_line_kernelI(DF16b|DF16_|Dh|f)Li(\d+)ELi(\d+)ELb([01])ELi(\d+)ELb([01])E", name)
    if m:
        dtype = {"DF16b": "bf16", "DF16_": "f16", "Dh": "f16", "f": "f32"}[m.group(1)]
        flag = lambda b: "true" if b == "1" else "false"
        return f"grouped_gemm_line_kernel<{dtype}, {m.group(2)}, {m.group(3)}, {flag(m.group(4))}, {m.group(5)}, {flag(m.group(6))}>"
    m = re.search(r"grouped_gemm_line_kernel<(.*?)>\(", name + "(")
    if m:
        args = [a.strip() for a in m.group(1).split(",")]
        if args[:3] == ["bool _Accum", "int", "E"]:  # the mis-demangled (bf16, 1)
            args = ["bf16", "1"] + args[3:]
        args[0] = {"__hip_bfloat16": "bf16", "__bf16": "bf16", "_Float16": "f16", "__half": "f16"}.get(args[0], args[0])
        return "grouped_gemm_line_kernel<" + ", ".join(args) + ">"
    return name


def load_traffic_summary(path: str = TRAFFIC_SUMMARY) -> dict:
    """kernel name (canonical_kernel_name) -> HBM bytes per launch, from the summary's tab-separated lines
    `kernel<TAB>launches<TAB>fetch KiB per launch (scaled)<TAB>write KiB per launch (scaled)<TAB>name in the counter file`."""
    table = {}
    if not os.path.exists(path):
        return table
    with open(path) as f:
        for line in f:
            if line.startswith("#") or not line.strip():
                continue
            name, _launches, fetch_kib, write_kib = line.rstrip("\n").split("\t")[:4]
            table[canonical_kernel_name(name)] = (float(fetch_kib) + float(write_kib)) * 1024.0
    return table


def summarize_pmc(fetch_dir: str, write_dir: str, out_path: str = TRAFFIC_SUMMARY) -> None:
    """Reduce the counter_collection.csv files of two rocprofv3 --pmc runs of this benchmark with --copy-calibration
    (FETCH_SIZE in one, WRITE_SIZE in the other) to one line per kernel: mean KiB per launch, each counter scaled by
    what it reads for the 1 GiB device copy of the same run (known size: 2^20 KiB each way)."""
    import csv
    import glob

    def per_kernel(directory: str, counter: str) -> dict:
        sums: dict = {}  # name -> [sum, launches, largest single reading]
        for path in glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True):
            with open(path, newline="") as f:
                for row in csv.DictReader(f):
                    if row.get("Counter_Name") != counter:
                        continue
                    rec = sums.setdefault(row["Kernel_Name"], [0.0, 0, 0.0])
                    value = float(row["Counter_Value"])
                    rec[0] += value
                    rec[1] += 1
                    rec[2] = max(rec[2], value)
        return sums

    def copy_factor(sums: dict, what: str) -> float:
        # the calibration copy (2^30 bytes, torch's device-to-device copy) is the largest single launch among the kernels
        # whose name says "copy" (the runtime's copyBuffer kernel also serves every small copy of the run)
        cands = [v[2] for k, v in sums.items() if "copy" in k.lower()]
        if not cands or max(cands) < float(1 << 18):
            raise SystemExit(f"no 1 GiB copy in the {what} run: was bench.py run with --copy-calibration?")
        return float(1 << 20) / max(cands)

    fetch, write = per_kernel(fetch_dir, "FETCH_SIZE"), per_kernel(write_dir, "WRITE_SIZE")
    ff, wf = copy_factor(fetch, "FETCH_SIZE"), copy_factor(write, "WRITE_SIZE")
    with open(out_path, "w") as f:
        f.write("# HBM traffic per launch of the grouped GEMM kernels in `python bench.py --copy-calibration` (C3 workload)\n")
        f.write(f"# from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (KiB per dispatch), scaled by {ff:.3f} and {wf:.3f}:\n")
        f.write("# what makes the same counter read 2^20 KiB for the run's own 1 GiB device copy\n")
        f.write("# kernel\tlaunches\tfetch_KiB_per_launch\twrite_KiB_per_launch\tname_in_the_counter_file\n")
        for name in sorted(fetch, key=canonical_kernel_name):
            if "grouped_gemm" not in name or name not in write:
                continue
            fv, wv = fetch[name], write[name]
            f.write(f"{canonical_kernel_name(name)}\t{fv[1]}\t{fv[0] / fv[1] * ff:.1f}\t{wv[0] / wv[1] * wf:.1f}\t{name}\n")
    print(f"wrote {out_path}")


# the kernel instantiation each launch name runs at this workload, as rocprofv3's kernel trace spells it
# (grouped_gemm_line_kernel<T, MODE, BN, BT, WGM, EXTRA>: MODE 0 grouped, 1 scatter, 2 swiglu, 4 dw; BT: contraction-strided
# operands; WGM = 2: four waves, one per SIMD; EXTRA: bias / side outputs)
ROCPROF_KERNEL = {
    "grouped_gemm_dw_rows": "grouped_gemm_line_kernel<bf16, 4, 256, true, 2, false>",
    "grouped_gemm<swiglu>": "grouped_gemm_line_kernel<bf16, 2, 256, false, 2, false>",
    "grouped_gemm_nn<scatter>": "grouped_gemm_line_kernel<bf16, 1, 256, true, 2, false>",
    "grouped_gemm_nn<grouped>": "grouped_gemm_line_kernel<bf16, 0, 256, true, 2, false>",
    "grouped_gemm<scatter>": "grouped_gemm_line_kernel<bf16, 1, 256, false, 2, false>",
}


def traffic_for(launch_name: str, summary_path: str = TRAFFIC_SUMMARY):
    """HBM bytes per launch of the kernel behind `launch_name`, or None when the tracked counter summary does not hold
    that kernel (spelled as rocprofv3 spells it, template arguments included)."""
    want = ROCPROF_KERNEL.get(launch_name)
    if want is None:
        return None
    return load_traffic_summary(summary_path).get(want)

# workload: configs[2] of the baseline, the configuration its headline metric (MoE fwd+bwd TFLOP/s) is quoted on
T, H, E, TOP_K, I = 16384, 4096, 8, 2, 14336
SEED = 42


def zipf_bias(logits, k: int, s: float = 1.0):
    """Per-expert additive logit bias c*log(1/rank) with c chosen so the routed load is closest to Zipf(s)."""
    import torch

    E_ = logits.size(1)
    ranks = torch.arange(1, E_ + 1, device=logits.device, dtype=torch.float32)
    target = (1.0 / ranks**s) / (1.0 / ranks**s).sum()
    best = None
    for c in [x * 0.05 for x in range(0, 81)]:
        bias = -c * torch.log(ranks)
        sel = (logits.float() + bias).topk(k, dim=-1).indices.flatten()
        freq = torch.bincount(sel, minlength=E_).float()
        freq = freq / freq.sum()
        err = float((freq - target).abs().sum())
        if best is None or err < best[0]:
            best = (err, c, bias, freq)
    return best[2], best[3], best[1]


def build_layer(dev, reverse_load: bool = False):
    import torch

    import cute_kernels

    torch.manual_seed(SEED)
    moe = cute_kernels.MoE(E, TOP_K, H, I, cute_kernels.swiglu_packed_cute, True, False, 0.02)
    moe = moe.to(torch.bfloat16).to(dev)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(SEED)).to(torch.bfloat16).to(dev)
    with torch.no_grad():
        bias, freq, c = zipf_bias(moe.gate(x), TOP_K, 1.0)
    if reverse_load:  # the same loads with the heaviest expert last (a measurement of tile-order robustness)
        bias, freq = bias.flip(0), freq.flip(0)
    bias = bias.to(torch.bfloat16)
    # the router has no bias parameter (torch_implementation.py:83 of the reference): skew goes in through a hook
    moe.gate.register_forward_hook(lambda mod, inp, out: out + bias)
    moe.zipf_logit_bias = bias
    grad_out = torch.randn(T, H, generator=torch.Generator().manual_seed(SEED + 1)).to(torch.bfloat16).to(dev)
    return moe, x, grad_out, freq.tolist(), c


def step(moe, x, grad_out):
    for p in moe.parameters():
        p.grad = None
    x.grad = None
    y, _ = moe(x)
    y.backward(grad_out)


def cpu_baseline(moe_gpu, bias_fn_freq, sample_tokens: int = T):
    """The torch CPU path (restated in oracle/moe_oracle.py) on `sample_tokens` tokens of the same layer (default: the
    whole batch, one forward+backward, 10 to 20 s on 16 host threads), same router skew."""
    import torch
    import torch.nn.functional as F

    from oracle import moe_oracle as mo

    oracle = mo.MoEOracle(E, TOP_K, H, I, mo.swiglu_packed_torch, True, False, 0.02).to(torch.bfloat16)
    oracle.load_state_dict({k: v.cpu() for k, v in moe_gpu.state_dict().items()})
    cpu_bias = moe_gpu.zipf_logit_bias.cpu()
    oracle.gate.register_forward_hook(lambda mod, inp, out: out + cpu_bias)
    xs = torch.randn(sample_tokens, H, generator=torch.Generator().manual_seed(SEED)).to(torch.bfloat16).requires_grad_()
    g = torch.randn(sample_tokens, H, generator=torch.Generator().manual_seed(SEED + 1)).to(torch.bfloat16)
    warm = xs[:32].detach().clone().requires_grad_()
    oracle(warm)[0].backward(g[:32])
    for p in oracle.parameters():
        p.grad = None
    t0 = time.perf_counter()
    y, _ = oracle(xs)
    y.backward(g)
    dt = time.perf_counter() - t0
    flops = 18.0 * sample_tokens * TOP_K * H * I
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"1 fwd+bwd of the same layer on T={sample_tokens} tokens (of {T}), bf16, same Zipf router bias, {dt:.2f} s; "
        f"os.cpu_count()={os.cpu_count()}",
    }


def secondary_hbm_kernels(dev):
    """count+scatter GB/s: the HBM-bound kernels on their own, algorithmic bytes / event time."""
    import torch

    import cute_kernels
    from cute_kernels import scattermoe

    def timed(fn, iters=20):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(iters):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / iters * 1e-3

    from cute_kernels import _C

    out = {}
    g = torch.Generator().manual_seed(SEED)
    lib = _C.lib()
    for n in (1 << 16, 1 << 22, 1 << 28):
        ids = torch.randint(0, 64, (n,), generator=g, dtype=torch.int32).to(dev) if n <= (1 << 22) else torch.randint(0, 64, (n,), dtype=torch.int32, device=dev)
        # straight through the C ABI with caller-owned outputs, as a C caller would (no Python-side allocation in the loop)
        counts, ends, starts = (torch.empty(64, dtype=torch.uint32, device=dev) for _ in range(3))
        ws = torch.zeros(lib.ck_count_workspace_words(64), dtype=torch.int32, device=dev)
        stream = torch.cuda.current_stream().cuda_stream

        def count():
            _C.check(lib.ck_count_offsets(ids.data_ptr(), 0, n, 64, counts.data_ptr(), ends.data_ptr(), starts.data_ptr(),
                                          ws.data_ptr(), stream))

        dt = timed(count, iters=200 if n <= (1 << 22) else 20)
        assert int(ends[-1]) == n
        b = 4 * n + 8 * 64 + 4 * 64
        out[f"count_offsets_N{n}_E64"] = {"us": dt * 1e6, "GB/s": b / dt / 1e9, "frac_hbm": b / dt / 1e9 / PEAK_HBM_GBS}
        del ids
    # C2 routing bookkeeping: logits [16384, 64] bf16, top-2 -> ids, gates, stable sort, counts / offsets.
    # Straight through the C ABI with caller-owned outputs (three launches: route, sort histogram + scan, sort scatter).
    Tr, Er, kr = 16384, 64, 2
    Rr = Tr * kr
    logits = torch.randn(Tr, Er, generator=g).to(torch.bfloat16).to(dev)
    i32 = dict(dtype=torch.int32, device=dev)
    sel, gates = torch.empty(Tr, kr, **i32), torch.empty(Tr, kr, dtype=torch.float32, device=dev)
    max_rows = lib.ck_sort_max_rows(Rr, Er, 128)
    se, ss = torch.empty(Rr, **i32), torch.empty(Rr, **i32)
    cnt, en, st = (torch.empty(Er, dtype=torch.uint32, device=dev) for _ in range(3))
    seg_starts, row_slot, tile_expert = torch.empty(Er + 1, **i32), torch.empty(max_rows, **i32), torch.empty(max_rows // 128, **i32)
    ws2 = torch.zeros(lib.ck_sort_workspace_words(Rr, Er), **i32)
    stream = torch.cuda.current_stream().cuda_stream

    def routing():
        _C.check(lib.ck_route_topk_softmax(logits.data_ptr(), _C.CK_BF16, Tr, Er, kr, sel.data_ptr(), gates.data_ptr(), None, stream))
        _C.check(lib.ck_sort_by_expert(sel.data_ptr(), 0, Rr, Er, 128, se.data_ptr(), ss.data_ptr(), cnt.data_ptr(), en.data_ptr(),
                                       st.data_ptr(), seg_starts.data_ptr(), row_slot.data_ptr(), tile_expert.data_ptr(),
                                       ws2.data_ptr(), stream))

    dt = timed(routing, iters=200)
    assert int(en[-1]) == Rr
    b = 2 * Tr * Er + 4 * 4 * Rr + 8 * Er
    out["route_sort_C2"] = {"us": dt * 1e6, "GB/s": b / dt / 1e9, "frac_hbm": b / dt / 1e9 / PEAK_HBM_GBS}
    # row gather / gated combine at the C3 shape
    R = T * TOP_K
    src = torch.randn(T, H, device=dev, dtype=torch.bfloat16)
    idx = torch.randperm(R, device=dev).to(torch.int32)
    dt = timed(lambda: cute_kernels.gather_rows(src, idx, None, TOP_K))
    b = 2 * R * H * 2
    out["gather_rows_C3"] = {"us": dt * 1e6, "GB/s": b / dt / 1e9, "frac_hbm": b / dt / 1e9 / PEAK_HBM_GBS}
    expanded = torch.randn(R, H, device=dev, dtype=torch.bfloat16)
    gates = torch.rand(T, TOP_K, device=dev, dtype=torch.bfloat16)
    dt = timed(lambda: scattermoe._combine(expanded, gates, T, TOP_K, H))
    b = R * H * 2 + T * H * 2 + 2 * R
    out["combine_rows_C3"] = {"us": dt * 1e6, "GB/s": b / dt / 1e9, "frac_hbm": b / dt / 1e9 / PEAK_HBM_GBS}
    del src, idx, expanded, gates

    # stand-alone SwiGLU (packed, C3 rows x 2I), RMSNorm and the fused residual add (C5 rows: 65,536 x 4,096), forward and
    # backward: straight through the C ABI with caller-owned outputs and workspaces, like the count rows above (through
    # autograd, a row would also time the allocator: 1.9 GB of fresh gradients per iteration)
    def rec(name, dt, b):
        out[name] = {"us": dt * 1e6, "GB/s": b / dt / 1e9, "frac_hbm": b / dt / 1e9 / PEAK_HBM_GBS}

    bf = _C.CK_BF16
    xp = torch.randn(R, 2 * I, device=dev, dtype=torch.bfloat16)
    yp = torch.empty(R, I, device=dev, dtype=torch.bfloat16)
    up_p, gate_p = xp[:, :I], xp[:, I:]  # packed order: up first, gate second
    rec("swiglu_packed_fwd_C3",
        timed(lambda: _C.check(lib.ck_swiglu_fwd(gate_p.data_ptr(), 2 * I, up_p.data_ptr(), 2 * I, yp.data_ptr(), I, R, I, bf, stream))),
        3 * R * I * 2)
    gy = torch.randn(R, I, device=dev, dtype=torch.bfloat16)
    dxp = torch.empty_like(xp)
    d_up, d_gate = dxp[:, :I], dxp[:, I:]
    rec("swiglu_packed_bwd_C3",
        timed(lambda: _C.check(lib.ck_swiglu_bwd(gate_p.data_ptr(), 2 * I, up_p.data_ptr(), 2 * I, gy.data_ptr(), I, d_gate.data_ptr(),
                                                 2 * I, d_up.data_ptr(), 2 * I, R, I, bf, stream))),
        5 * R * I * 2)
    del xp, yp, gy, dxp, up_p, gate_p, d_up, d_gate
    Bn, Hn = 65536, 4096
    xn = torch.randn(Bn, Hn, device=dev, dtype=torch.bfloat16)
    wn = torch.ones(Hn, device=dev, dtype=torch.bfloat16)
    yn, gn, dxn = torch.empty_like(xn), torch.randn_like(xn), torch.empty_like(xn)
    rstd = torch.empty(Bn, device=dev, dtype=torch.float32)
    dwn = torch.empty(Hn, device=dev, dtype=torch.float32)
    partial = torch.empty(max(lib.ck_rmsnorm_bwd_partial_rows(Bn), 1), Hn, device=dev, dtype=torch.float32)
    rec("rmsnorm_fwd_C5",
        timed(lambda: _C.check(lib.ck_rmsnorm_fwd(xn.data_ptr(), wn.data_ptr(), 1e-6, Bn, Hn, yn.data_ptr(), rstd.data_ptr(), bf, stream))),
        2 * Bn * Hn * 2 + 4 * Bn)
    rec("rmsnorm_bwd_C5",
        timed(lambda: _C.check(lib.ck_rmsnorm_bwd(xn.data_ptr(), wn.data_ptr(), gn.data_ptr(), rstd.data_ptr(), 1e-6, Bn, Hn,
                                                  dxn.data_ptr(), partial.data_ptr(), dwn.data_ptr(), bf, stream))),
        3 * Bn * Hn * 2 + 4 * Bn)
    # the step that precedes an MoE block in a transformer: residual add fused into the norm (same rows); algorithmic
    # bytes: forward reads x, residual and writes y, added; backward reads added, d_y, d_added and writes d_x, d_residual
    rn, an, ga, drn = torch.randn_like(xn), torch.empty_like(xn), torch.randn_like(xn), torch.empty_like(xn)
    rec("fused_residual_add_rmsnorm_fwd_C5",
        timed(lambda: _C.check(lib.ck_fused_residual_add_rmsnorm_fwd(xn.data_ptr(), rn.data_ptr(), wn.data_ptr(), 1e-6, 1.0, Bn, Hn,
                                                                     yn.data_ptr(), an.data_ptr(), rstd.data_ptr(), bf, stream))),
        4 * Bn * Hn * 2 + 4 * Bn)
    rec("fused_residual_add_rmsnorm_bwd_C5",
        timed(lambda: _C.check(lib.ck_fused_residual_add_rmsnorm_bwd(an.data_ptr(), wn.data_ptr(), gn.data_ptr(), ga.data_ptr(),
                                                                     rstd.data_ptr(), 1e-6, 1.0, Bn, Hn, dxn.data_ptr(), drn.data_ptr(),
                                                                     partial.data_ptr(), dwn.data_ptr(), bf, stream))),
        5 * Bn * Hn * 2 + 4 * Bn)
    # multiplier 1: both gradients are the same values and one buffer takes them (the Python wrapper's call)
    rec("fused_residual_add_rmsnorm_bwd_one_buffer_C5",
        timed(lambda: _C.check(lib.ck_fused_residual_add_rmsnorm_bwd(an.data_ptr(), wn.data_ptr(), gn.data_ptr(), ga.data_ptr(),
                                                                     rstd.data_ptr(), 1e-6, 1.0, Bn, Hn, dxn.data_ptr(), dxn.data_ptr(),
                                                                     partial.data_ptr(), dwn.data_ptr(), bf, stream))),
        4 * Bn * Hn * 2 + 4 * Bn)
    del yn, gn, dxn, rn, an, ga, drn, partial
    # RMSNorm fused ahead of the router (one pass: normalised rows + router logits, optionally the e4m3 rows) against the
    # separate kernels (rmsnorm, the router's linear layer on the BLAS library, the row quantiser); algorithmic bytes:
    # rows in and out once, logits out (+ 1 byte per element and a scale per row with the e4m3 rows)
    for tag, (Bp, Hp, Ep) in {"C4": (8192, 2048, 64), "C5": (65536, 4096, 128)}.items():
        xr_, wr_ = xn[:Bp, :Hp].contiguous(), wn[:Hp].contiguous()
        gr_ = (torch.randn(Ep, Hp, device=dev) * Hp**-0.5).to(torch.bfloat16)
        b_plain, b_quant = 2 * Bp * Hp * 2 + Bp * Ep * 2, 2 * Bp * Hp * 2 + Bp * Ep * 2 + Bp * Hp + 4 * Bp
        with torch.no_grad():
            rec(f"rmsnorm_route_{tag}", timed(lambda: cute_kernels.rmsnorm_route_cute(xr_, wr_, gr_, 1e-6, fused=True)), b_plain)
            rec(f"rmsnorm_route_e4m3_{tag}", timed(lambda: cute_kernels.rmsnorm_route_cute(xr_, wr_, gr_, 1e-6, quantize=True, fused=True)), b_quant)
            rec(f"rmsnorm_then_linear_{tag}", timed(lambda: cute_kernels.rmsnorm_route_cute(xr_, wr_, gr_, 1e-6, fused=False)), b_plain)
            rec(f"rmsnorm_then_linear_then_quant_{tag}", timed(lambda: cute_kernels.rmsnorm_route_cute(xr_, wr_, gr_, 1e-6, quantize=True, fused=False)), b_quant)
        del xr_, wr_, gr_
    del xn, wn
    # router-logit statistics: softmax over all experts at the C5 router shape (65,536 x 128)
    lg = torch.randn(Bn, 128, device=dev, dtype=torch.bfloat16)
    sm, gs, dlg = torch.empty_like(lg), torch.randn_like(lg), torch.empty_like(lg)
    rec("softmax_fwd_C5_router",
        timed(lambda: _C.check(lib.ck_softmax_fwd(lg.data_ptr(), 1.0, Bn, 128, sm.data_ptr(), bf, stream)), iters=100), 2 * Bn * 128 * 2)
    rec("softmax_bwd_C5_router",
        timed(lambda: _C.check(lib.ck_softmax_bwd(sm.data_ptr(), gs.data_ptr(), 1.0, Bn, 128, dlg.data_ptr(), bf, stream)), iters=100),
        3 * Bn * 128 * 2)
    del lg, sm, gs, dlg
    torch.cuda.empty_cache()

    # C4: fine-grained MoE fwd+bwd behind an RMSNorm prologue (T=8192, H=2048, E=64, top-8, I=1408, uniform routing)
    T4, H4, E4, K4, I4 = 8192, 2048, 64, 8, 1408
    torch.manual_seed(SEED)
    moe4 = cute_kernels.MoE(E4, K4, H4, I4, cute_kernels.swiglu_packed_cute, True, False, 0.02).to(torch.bfloat16).to(dev)
    w4 = (1 + 0.02 * torch.randn(H4, device=dev)).to(torch.bfloat16).requires_grad_()
    x4 = torch.randn(T4, H4, device=dev, dtype=torch.bfloat16, requires_grad=True)
    g4 = torch.randn(T4, H4, device=dev, dtype=torch.bfloat16)

    def step4():
        for p_ in moe4.parameters():
            p_.grad = None
        x4.grad = None
        w4.grad = None
        y4, _ = moe4.forward_with_norm(x4, w4, 1e-6)  # the norm fused ahead of the router: one kernel for rows + logits
        y4.backward(g4)

    dt = timed(step4, iters=10)
    f4 = 18.0 * T4 * K4 * H4 * I4
    configs = {}
    configs["C4_moe_fwd_bwd"] = {"ms": dt * 1e3, "TFLOP/s": f4 / dt / 1e12, "frac_mfma": f4 / dt / 1e12 / PEAK_BF16_TFLOPS}
    del moe4, w4, x4, g4
    torch.cuda.empty_cache()

    # C5: quantised-expert forward (e4m3 weights, per-channel scales; activations e4m3 per token) behind an RMSNorm
    # prologue: T=65,536, H=4,096, E=128, top-8, I=1,536, Zipf(0.8) load, forward only
    T5, H5, E5, K5, I5 = 65536, 4096, 128, 8, 1536
    torch.manual_seed(SEED)
    moe5 = cute_kernels.MoE(E5, K5, H5, I5, cute_kernels.swiglu_packed_cute, True, False, 0.02).to(torch.bfloat16).to(dev)
    x5 = torch.randn(T5, H5, device=dev, dtype=torch.bfloat16)
    w5 = (1 + 0.02 * torch.randn(H5, device=dev)).to(torch.bfloat16)
    with torch.no_grad():
        bias5, freq5, c5 = zipf_bias(moe5.gate(cute_kernels.rmsnorm_cute(x5[:16384], w5, 1e-6)), K5, 0.8)
    bias5 = bias5.to(torch.bfloat16)
    moe5.gate.register_forward_hook(lambda mod, inp, o: o + bias5)
    q5 = cute_kernels.MoE_E4M3(moe5)
    moe5.c_fc.weight.data = torch.empty(0, device=dev)  # the 16-bit expert weights are not part of the fp8 layer
    moe5.c_proj.weight.data = torch.empty(0, device=dev)
    torch.cuda.empty_cache()

    def step5():
        with torch.no_grad():  # separate norm: at E * H = 128 * 4096 the one-pass prologue kernel does not pay (see the
            q5(cute_kernels.rmsnorm_cute(x5, w5, 1e-6))  # rmsnorm_route_* lines), and the Zipf bias enters through the gate's hook

    dt = timed(step5, iters=5)
    timer = scattermoe.LaunchTimer()
    scattermoe.launch_timer = timer
    step5()
    scattermoe.launch_timer = None
    torch.cuda.synchronize()
    f5 = 6.0 * T5 * K5 * H5 * I5
    launches = {}
    for name, dims, s_, e_ in timer.records:
        ms = s_.elapsed_time(e_)
        fl = 2.0 * T5 * K5 * dims[0] * dims[1]
        launches[name] = {"N_K": list(dims), "ms": ms, "TFLOP/s": fl / ms / 1e9, "frac_mfma_fp8": fl / ms / 1e9 / PEAK_FP8_TFLOPS}
    configs["C5_moe_e4m3_fwd"] = {"ms": dt * 1e3, "TFLOP/s": f5 / dt / 1e12, "frac_mfma_fp8": f5 / dt / 1e12 / PEAK_FP8_TFLOPS,
                              "zipf_c": c5, "max_expert_share": max(freq5.tolist()), "launches": launches}
    return out, configs


def gemm_only(dev, launches: int, stamps: bool = False, zeros: bool = False):
    """Just the c_fc-forward-shape grouped GEMM (grouped epilogue) at the C3 shape: the target of counter runs.
    stamps: with a CK_STAMP measurement build (build.py --define CK_STAMP=1 --output FILE.so, loaded with --lib FILE.so),
    also print where a wave's cycles go: main loop, waiting for loads, waiting at the barrier, epilogue.
    zeros: all-zero operands (the chip's clock under the same instruction stream)."""
    import numpy as np
    import torch

    import cute_kernels
    from cute_kernels import _C, scattermoe

    R = T * TOP_K
    p = 1.0 / np.arange(1, E + 1)
    ids = torch.from_numpy(np.random.default_rng(SEED).choice(E, size=R, p=p / p.sum())).to(torch.int32)
    seg = cute_kernels.sort_by_expert(ids.to(dev), E, 256)
    x = torch.randn(T, H, device=dev, dtype=torch.bfloat16)
    w = torch.randn(E, 2 * I, H, device=dev, dtype=torch.bfloat16) * 0.02
    if zeros:
        x.zero_()
        w.zero_()
    y = torch.empty(seg.max_rows, 2 * I, device=dev, dtype=torch.bfloat16)
    trace = None
    if stamps:
        trace = torch.zeros(8 * 8 * 20000, dtype=torch.int64, device=dev)
        _C.set_option("trace_buffer", trace.data_ptr())  # stamp builds write their per-wave cycle counts here
    for _ in range(2):
        scattermoe._gemm(x, TOP_K, w, seg, _C.CK_EPI_GROUPED, y)
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(launches):
        scattermoe._gemm(x, TOP_K, w, seg, _C.CK_EPI_GROUPED, y)
    e.record()
    torch.cuda.synchronize()
    ms = s.elapsed_time(e) / launches
    flops = 4.0 * R * H * I
    rec = {"kernel": "grouped_gemm<grouped>", "shape": [R, 2 * I, H], "avg_launch_ms": ms,
           "TFLOP/s": flops / ms / 1e9, "frac_mfma": flops / ms / 1e9 / PEAK_BF16_TFLOPS}
    if trace is not None:
        t = trace.view(-1, 8).cpu().numpy().astype(np.float64)
        t = t[t[:, 5] > 0]  # waves that ran a main loop
        assert len(t) > 0, "no stamps: is --lib a CK_STAMP build?"
        tot = t[:, 0] + t[:, 1] + t[:, 4]
        rec["stamps"] = {
            "waves": int(len(t)), "k_steps": float(t[:, 5].mean()),
            "cycles_per_wave": {"prologue": float(t[:, 0].mean()), "main_loop": float(t[:, 1].mean()),
                                "load_wait": float(t[:, 2].mean()), "barrier_wait": float(t[:, 3].mean()),
                                "epilogue": float(t[:, 4].mean()), "slice0_per_step": float((t[:, 6] / (t[:, 5] - 1)).mean()),
                                "slice1_per_step": float((t[:, 7] / (t[:, 5] - 1)).mean())},
            "share_of_tile": {"main_loop": float((t[:, 1] / tot).mean()), "load_wait": float((t[:, 2] / tot).mean()),
                              "barrier_wait": float((t[:, 3] / tot).mean()), "epilogue": float((t[:, 4] / tot).mean())},
            "main_loop_cycles_per_k_step": float((t[:, 1] / t[:, 5]).mean()),
        }
    print(json.dumps(rec))


def library_gemm_yardstick(dev, iters: int = 10):
    """What this box's chip sustains on dense bf16 products of the layer's per-expert shapes through torch.matmul
    (the vendor GEMM library), on the same kind of data (activations N(0,1), weights N(0,0.02)) and on zeros: the
    same-box yardstick for the grouped GEMM figures (clocks are power-managed and depend on the operand bits)."""
    import torch

    out = {}
    shapes = {
        "c_fc_largest_expert_10928x28672x4096": (10928, 2 * I, H),
        "c_proj_largest_expert_10928x4096x14336": (10928, H, I),
        "c_fc_all_rows_32768x28672x4096": (T * TOP_K, 2 * I, H),
        "square_8192": (8192, 8192, 8192),
    }
    for name, (m, n, k) in shapes.items():
        for data in ("normal", "zeros"):
            if data == "normal":
                a = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
                b = (torch.randn(n, k, device=dev) * 0.02).to(torch.bfloat16)
            else:
                a = torch.zeros(m, k, device=dev, dtype=torch.bfloat16)
                b = torch.zeros(n, k, device=dev, dtype=torch.bfloat16)
            c = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
            for _ in range(3):
                torch.matmul(a, b.t(), out=c)
            torch.cuda.synchronize()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(iters):
                torch.matmul(a, b.t(), out=c)
            e.record()
            torch.cuda.synchronize()
            ms = s.elapsed_time(e) / iters
            tf = 2.0 * m * n * k / ms / 1e9
            out[f"{name}_{data}"] = {"ms": ms, "TFLOP/s": tf, "frac_mfma": tf / PEAK_BF16_TFLOPS}
            del a, b, c
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--skip-cpu-baseline", action="store_true")
    ap.add_argument("--skip-secondary", action="store_true")
    ap.add_argument("--only-gemm", type=int, default=0, metavar="LAUNCHES",
                    help="run only the c_fc-forward-shape grouped GEMM this many times (for rocprofv3 --pmc runs)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device copy (outside the timed region): the known-size kernel that "
                    "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--lib", default=None, metavar="FILE.so",
                    help="load this build of the library (a measurement build from build.py --define ... --output) instead of the product one")
    ap.add_argument("--zeros", action="store_true", help="with --only-gemm: all-zero operands")
    ap.add_argument("--reverse-load", action="store_true",
                    help="the C3 step with the expert loads reversed (heaviest expert last); not the headline workload")
    ap.add_argument("--no-split", action="store_true", help="never split the last round of GEMM tiles (A/B measurement)")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="ck_debug_set_option(NAME, VALUE) before the run (A/B measurement of kernel variants)")
    ap.add_argument("--summarize-pmc", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="no GPU work: reduce two rocprofv3 --pmc output directories to profiles/grouped_gemm_c3_hbm_traffic.txt")
    ap.add_argument("--stamps", action="store_true",
                    help="with --only-gemm and a CK_STAMP measurement build: print the per-wave cycle breakdown")
    ap.add_argument("--only-yardstick", action="store_true",
                    help="run only torch.matmul on the layer's per-expert shapes (the same-box library yardstick)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build uses no second GPU (no collectives, no sharding); run with --gpus 1",
              file=sys.stderr)
        return 2

    if args.summarize_pmc:
        summarize_pmc(*args.summarize_pmc)
        return 0

    import torch

    from cute_kernels import _C, scattermoe

    if args.lib:
        _C.use_library(args.lib)
    if args.no_split:
        scattermoe.options.gemm_split = False
    for item in args.option:
        name, _, value = item.partition("=")
        _C.set_option(name, int(value))
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    if args.only_gemm > 0:
        gemm_only(dev, args.only_gemm, args.stamps, args.zeros)
        return 0
    if args.only_yardstick:
        print(json.dumps({"library_gemm_yardstick": library_gemm_yardstick(dev)}))
        return 0
    moe, x, grad_out, freq, zipf_c = build_layer(dev, args.reverse_load)
    x.requires_grad_()

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 2^30 B, writes 2^30 B
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step(moe, x, grad_out)
    torch.cuda.synchronize()

    timer = scattermoe.LaunchTimer()
    scattermoe.launch_timer = timer
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(moe, x, grad_out)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    scattermoe.launch_timer = None

    R = T * TOP_K
    flops_step = 18.0 * R * H * I
    value = flops_step / dt / 1e12

    # per-kernel launch durations from the events recorded inside the timed region
    per_kernel: dict = {}
    for name, dims, s, e in timer.records:
        rec = per_kernel.setdefault(name, {"ms": 0.0, "launches": 0, "flops": 0.0})
        rec["ms"] += s.elapsed_time(e)
        rec["launches"] += 1
        rec["flops"] += 2.0 * R * dims[0] * dims[1]  # 2*R*N*K (forward shapes) or 2*R*M*N (weight gradients)
    dominant = max(per_kernel, key=lambda n: per_kernel[n]["ms"])
    d = per_kernel[dominant]
    achieved = d["flops"] / (d["ms"] * 1e-3) / 1e12
    roofline = {
        "bound": "mfma",
        "kernel": dominant,
        "rocprof_kernel": ROCPROF_KERNEL.get(dominant),
        "achieved": achieved,
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": achieved / PEAK_BF16_TFLOPS,
        "traffic": traffic_for(dominant),
        "traffic_source": "profiles/grouped_gemm_c3_hbm_traffic.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, "
        "matched by kernel name (null: that kernel is not in the summary); not measured in this run",
        "avg_launch_ms": d["ms"] / d["launches"],
        "flops_per_launch": d["flops"] / d["launches"],
    }
    kernels = {
        n: {
            "avg_launch_ms": r["ms"] / r["launches"],
            "launches_per_step": r["launches"] / args.steps,
            "TFLOP/s": r["flops"] / (r["ms"] * 1e-3) / 1e12,
            "frac_mfma": r["flops"] / (r["ms"] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        }
        for n, r in per_kernel.items()
    }
    gemm_ms_per_step = sum(r["ms"] for r in per_kernel.values()) / args.steps

    line = {
        "metric": "MoE fwd+bwd TFLOP/s",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "C3 Mixtral-shape MoE layer fwd+bwd: T=16384 H=4096 E=8 top-2 I=14336 SwiGLU, Zipf(1.0) load"
            + (" REVERSED (heaviest expert last)" if args.reverse_load else ""),
            "routed_rows": R,
            "flops_per_step": flops_step,
            "expert_load": [round(f, 4) for f in freq],
            "zipf_bias_scale": zipf_c,
        },
        "frac_mfma_peak": value / PEAK_BF16_TFLOPS,
        "gemm_ms_per_step": gemm_ms_per_step,
        "roofline": roofline,
        "kernels": kernels,
    }
    if not args.skip_secondary:
        del moe, x, grad_out
        torch.cuda.empty_cache()
        # the secondary metric (count + scatter GB/s: the HBM-bound kernels on their own) and the other two GPU configs
        line["count_scatter"], line["other_configs"] = secondary_hbm_kernels(dev)
        line["library_gemm_yardstick"] = library_gemm_yardstick(dev)
        moe = None
    if not args.skip_cpu_baseline:
        if moe is None:
            moe = build_layer(dev)[0]
        line["cpu_baseline"] = cpu_baseline(moe, None)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

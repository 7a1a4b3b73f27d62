#!/usr/bin/env python3
"""Headline benchmark: BF16 M-grouped GEMM, G=128, M=655360, N=1536, K=2048 on one MI355X.

One "step" is one pass of the hot path (one ``m_grouped_gemm`` launch) over a synthetic batch whose
operands are already resident in HBM.  Prints ONE JSON line: TFLOP/s = 2*M*N*K / time, the MFMA
roofline fraction of the GEMM kernel (HIP-event timed on the launch stream) and, beside it, the
reference's per-group torch matmul timed on this box's host cores over a bounded sample of groups.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]
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

PEAK_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0}   # MI355X dense MFMA peaks
PEAK_HBM_GBS = 8000.0

# HBM-side bytes per launch of each workload's kernel in GB, measured offline with rocprofv3
# (--pmc FETCH_SIZE and --pmc WRITE_SIZE, one counter per run, each scaled by what the counter reads for a
# plain 1 GiB device copy: x2.0 and x1.0).  The runs and their figures are listed in profiles/hbm_traffic.txt.
# FETCH_SIZE includes L2 fills served by the memory-side cache, so these are upper bounds on DRAM traffic.
MEASURED_TRAFFIC_GB = {
    "bf16_m_grouped_gateup_nt": 11.71,
    "bf16_m_grouped_gateup_nn": 11.55,
    "bf16_m_grouped_gateup_fp8_out": 10.39,
    "bf16_m_grouped_down_nt": 5.50,
    "bf16_m_grouped_down_nn": 5.47,
    "bf16_masked_decode": 2.59,
    "bf16_k_grouped_wgrad": 34.00,
    "fp8_block_m_grouped": 26.44,
    "fp8_channel_m_grouped": 26.62,
    "fp8_channel_k_grouped": 18.37,
    "quant_trans128": 8.12,
    "moe_permute": 3.06,      # the row mover (the sort kernels move < 1 % of that)
    "moe_unpermute": 3.07,
}

G, M_TOTAL = 128, 655360
WORKLOADS = {
    # name: (kind, N, K, trans_b)
    "bf16_m_grouped_gateup_nt": ("mg", 1536, 2048, True),
    "bf16_m_grouped_gateup_nn": ("mg", 1536, 2048, False),
    "bf16_m_grouped_down_nt": ("mg", 2048, 768, True),
    "bf16_m_grouped_down_nn": ("mg", 2048, 768, False),
    "bf16_m_grouped_gateup_fp8_out": ("mgq", 1536, 2048, True),   # same GEMM, output quantised 1x128 in the epilogue
    "bf16_masked_decode": ("masked", 4096, 1536, True),
    "bf16_k_grouped_wgrad": ("kg", 4096, 3072, False),      # N_DIM, M_DIM
    "fp8_block_m_grouped": ("fp8", 3072, 4096, True),
    "fp8_channel_m_grouped": ("fp8c", 3072, 4096, True),     # per-token x per-channel scales, same shape
    "fp8_channel_k_grouped": ("fp8ck", 4096, 3072, False),   # N_DIM, M_DIM; tokens along K
    "quant_trans128": ("quant", 4096, 0, False),
    # MoE token movement either side of the GEMMs: 81920 tokens x top-8 = 655360 rows of 2048 bf16
    "moe_permute": ("permute", 2048, 8, False),       # hidden, topK
    "moe_unpermute": ("unpermute", 2048, 8, False),
}


def build_workload(name: str, dev, seed: int = 2026, zeros: bool = False, num_cu: int = -1):
    """Returns (fn, flops_per_step, algorithmic_bytes_per_step, dtype_tag, description, cpu_sample_fn); leaves a
    per-group library-GEMM loop over the same operands in ``build_workload.vendor_loop`` where one exists."""
    build_workload.vendor_loop = None
    from triton_grouped_gemm_amd import workloads as wl
    from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm
    kind, N, K, trans_b = WORKLOADS[name]
    sizes_cpu = wl.dirichlet_multinomial_sizes(G, M_TOTAL, 128, seed=seed)
    sizes = sizes_cpu.to(dev)
    if kind == "mg":
        a = wl.randn_bf16((M_TOTAL, K), K ** -0.5, seed + 1, dev)
        b = wl.randn_bf16((G, N, K) if trans_b else (G, K, N), K ** -0.5, seed + 2, dev)
        if zeros:  # same kernel, same traffic, no switching activity in the multipliers
            a.zero_()
            b.zero_()
        fn = lambda: m_grouped_gemm(a, b, sizes, trans_b, numSM=num_cu)
        flops = 2.0 * M_TOTAL * N * K
        nbytes = 2.0 * M_TOTAL * K + 2.0 * G * N * K + 2.0 * M_TOTAL * N

        def cpu_sample(budget_s: float):
            from oracle import gemm_ref
            order = torch.argsort(sizes_cpu, descending=True).tolist()
            starts = (sizes_cpu.cumsum(0) - sizes_cpu).tolist()
            done_flops, t_used, groups = 0.0, 0.0, 0
            warm = True
            for g in order:
                n = int(sizes_cpu[g])
                if n == 0:
                    continue
                ag = a[starts[g]:starts[g] + n].cpu()
                bg = b[g:g + 1].cpu()
                if warm:
                    gemm_ref.gmm(ag[:256], bg, [256], trans_b)
                    warm = False
                t0 = time.perf_counter()
                gemm_ref.gmm(ag, bg, [n], trans_b)
                t_used += time.perf_counter() - t0
                done_flops += 2.0 * n * N * K
                groups += 1
                if t_used >= budget_s:
                    break
            return done_flops / t_used / 1e12, f"{groups} largest groups of {G} ({done_flops / flops * 100:.1f}% of the step's flops), bf16 torch matmul per group"
        bounds = [(int(s0), int(s0 + n)) for s0, n in zip((sizes_cpu.cumsum(0) - sizes_cpu).tolist(), sizes_cpu.tolist())]
        c_ref = torch.empty((M_TOTAL, N), device=dev, dtype=torch.bfloat16)

        def vendor_loop():  # one library GEMM per expert, the GPU baseline the reference's tables compare against
            for g, (s0, s1) in enumerate(bounds):
                if s1 > s0:
                    torch.matmul(a[s0:s1], b[g].t() if trans_b else b[g], out=c_ref[s0:s1])
        build_workload.vendor_loop = vendor_loop
        return fn, flops, nbytes, "bf16", dict(workload=name, G=G, M=M_TOTAL, N=N, K=K, trans_b=trans_b,
                                               group_sizes="dirichlet-multinomial, 128-aligned", seed=seed), cpu_sample
    if kind == "mgq":
        from triton_grouped_gemm_amd.gemm.fused import m_grouped_gemm_fp8_out
        a = wl.randn_bf16((M_TOTAL, K), K ** -0.5, seed + 1, dev)
        b = wl.randn_bf16((G, N, K), K ** -0.5, seed + 2, dev)
        fn = lambda: m_grouped_gemm_fp8_out(a, b, sizes, trans_b, scales_mn_major=True)
        nbytes = 2.0 * M_TOTAL * K + 2.0 * G * N * K + 1.0 * M_TOTAL * N + 4.0 * M_TOTAL * N / 128
        return (fn, 2.0 * M_TOTAL * N * K, nbytes, "bf16",
                dict(workload=name, G=G, M=M_TOTAL, N=N, K=K, trans_b=trans_b, output="e4m3fn codes + 1x128 fp32 scales",
                     group_sizes="dirichlet-multinomial, 128-aligned", seed=seed), None)
    if kind == "masked":
        from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_masked_TMA import m_grouped_gemm_masked
        m_max = 512
        mm_cpu = wl.masked_counts(G, m_max, seed)
        mm = mm_cpu.to(dev)
        lhs = wl.randn_bf16((G * m_max, K), K ** -0.5, seed + 1, dev)
        rhs = wl.randn_bf16((G, N, K), K ** -0.5, seed + 2, dev)
        out = torch.empty((G * m_max, N), device=dev, dtype=torch.bfloat16)
        mv = float(mm_cpu.sum())
        fn = lambda: m_grouped_gemm_masked(lhs, rhs, out, mm, m_max)
        return (fn, 2.0 * mv * N * K, 2.0 * mv * K + 2.0 * int((mm_cpu > 0).sum()) * N * K + 2.0 * mv * N, "bf16",
                dict(workload=name, G=G, m_max=m_max, N=N, K=K, valid_rows=int(mv), seed=seed), None)
    if kind == "kg":
        from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm
        Nd, Md = N, K
        a = wl.randn_bf16((M_TOTAL, Md), 1.0, seed + 1, dev)
        b = wl.randn_bf16((M_TOTAL, Nd), 1.0, seed + 2, dev)
        fn = lambda: k_grouped_gemm(a, b, sizes)
        bounds = [(int(s0), int(s0 + n)) for s0, n in zip((sizes_cpu.cumsum(0) - sizes_cpu).tolist(), sizes_cpu.tolist())]
        c_ref = torch.zeros((G, Md, Nd), device=dev, dtype=torch.bfloat16)

        def vendor_loop():
            for g, (s0, s1) in enumerate(bounds):
                if s1 > s0:
                    torch.matmul(a[s0:s1].t(), b[s0:s1], out=c_ref[g])
        build_workload.vendor_loop = vendor_loop
        return (fn, 2.0 * M_TOTAL * Md * Nd, 2.0 * M_TOTAL * (Md + Nd) + 2.0 * G * Md * Nd, "bf16",
                dict(workload=name, G=G, K_total=M_TOTAL, M_dim=Md, N_dim=Nd, seed=seed), None)
    if kind == "fp8":
        from triton_grouped_gemm_amd.gemm.deep_gemm_ops import m_grouped_fp8_nt_contiguous
        from triton_grouped_gemm_amd.quant.fp8_cast import per_block_cast_to_fp8, per_token_cast_to_fp8
        a = wl.randn_bf16((M_TOTAL, K), 1.0, seed + 1, dev)
        aq = per_token_cast_to_fp8(a, scales_mn_major=True)
        del a
        w = wl.randn_bf16((G, N, K), 1.0, seed + 2, dev)
        wq = per_block_cast_to_fp8(w)
        del w
        out = torch.empty((M_TOTAL, N), device=dev, dtype=torch.bfloat16)
        fn = lambda: m_grouped_fp8_nt_contiguous(aq, wq, sizes, out=out)
        nbytes = M_TOTAL * K + 4.0 * M_TOTAL * K / 128 + G * N * K + 4.0 * G * (N / 128) * (K / 128) + 2.0 * M_TOTAL * N
        return (fn, 2.0 * M_TOTAL * N * K, nbytes, "fp8",
                dict(workload=name, G=G, M=M_TOTAL, N=N, K=K, recipe="1x128 act / 128x128 weight, e4m3fn", seed=seed), None)
    if kind == "fp8c":
        from triton_grouped_gemm_amd.gemm.FP8.m_grouped_gemm_channel_expert import gmm_fp8_act_per_channel_w_per_expert
        gen = torch.Generator(device=dev).manual_seed(seed + 3)
        a = wl.randn_bf16((M_TOTAL, K), 1.0, seed + 1, dev).to(torch.float8_e4m3fn)
        w = wl.randn_bf16((G, N, K), 1.0, seed + 2, dev).to(torch.float8_e4m3fn)
        sa = torch.rand(M_TOTAL, 1, device=dev, generator=gen) + 0.5
        sb = torch.rand(G * N, device=dev, generator=gen) + 0.5
        fn = lambda: gmm_fp8_act_per_channel_w_per_expert(a, sa, w, sb, sizes, torch.bfloat16)
        nbytes = M_TOTAL * K + 4.0 * M_TOTAL + G * N * K + 4.0 * G * N + 2.0 * M_TOTAL * N
        return (fn, 2.0 * M_TOTAL * N * K, nbytes, "fp8",
                dict(workload=name, G=G, M=M_TOTAL, N=N, K=K, recipe="per-token x per-channel scales, e4m3fn", seed=seed), None)
    if kind == "fp8ck":
        from triton_grouped_gemm_amd.gemm.FP8.k_grouped_gemm_channel_expert import matmul as k_grouped_fp8
        m_dim, n_dim = K, N
        gen = torch.Generator(device=dev).manual_seed(seed + 3)
        x = wl.randn_bf16((m_dim, M_TOTAL), 1.0, seed + 1, dev).to(torch.float8_e4m3fn)
        y = wl.randn_bf16((n_dim, M_TOTAL), 1.0, seed + 2, dev).to(torch.float8_e4m3fn)
        xs = torch.rand(m_dim, G, device=dev, generator=gen) + 0.5
        ys = torch.rand(n_dim, G, device=dev, generator=gen) + 0.5
        fn = lambda: k_grouped_fp8(x, xs, y, ys, sizes, m_dim, n_dim, M_TOTAL, G)
        nbytes = 1.0 * M_TOTAL * (m_dim + n_dim) + 4.0 * G * (m_dim + n_dim) + 2.0 * G * m_dim * n_dim
        return (fn, 2.0 * M_TOTAL * m_dim * n_dim, nbytes, "fp8",
                dict(workload=name, G=G, M=m_dim, N=n_dim, K_total=M_TOTAL, recipe="per-channel x per-expert scales, e4m3fn",
                     seed=seed), None)
    if kind == "quant":
        from triton_grouped_gemm_amd.quant.trans_per_block_quant_expand_128x import trans_per_block_quant_expand_128x
        x = wl.randn_bf16((M_TOTAL, N), 1.0, seed + 1, dev)
        me = M_TOTAL + 128 * G - M_TOTAL % 128
        fn = lambda: trans_per_block_quant_expand_128x(x, sizes)
        nbytes = 2.0 * M_TOTAL * N + 1.0 * N * me + 4.0 * (N / 128) * (me / 128)
        return fn, 0.0, nbytes, "bf16->fp8", dict(workload=name, G=G, M=M_TOTAL, N=N, seed=seed), None
    if kind in ("permute", "unpermute"):
        from triton_grouped_gemm_amd import ops
        H, topk = N, K
        T = M_TOTAL // topk
        gen = torch.Generator(device="cpu").manual_seed(seed)
        # each token picks topk distinct experts (random scores, top-k), as a router would
        indices = torch.rand(T, G, generator=gen).topk(topk, dim=1).indices.to(torch.int32).to(dev)
        x = wl.randn_bf16((T, H), 1.0, seed + 1, dev)
        probs = torch.rand(T, topk, generator=gen).to(dev)
        if kind == "permute":
            fn = lambda: ops.permute(x, indices, num_experts=G)
            nbytes = 2.0 * T * H + 2.0 * T * topk * H + 4.0 * T * topk * 2
        else:
            perm, rmap = ops.permute(x, indices, num_experts=G)
            fn = lambda: ops.unpermute(perm, rmap, probs)
            nbytes = 2.0 * T * topk * H + 2.0 * T * H + 4.0 * T * topk * 2
        return fn, 0.0, nbytes, "bf16", dict(workload=name, tokens=T, topk=topk, hidden=H, experts=G, seed=seed), None
    raise ValueError(name)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="bf16_m_grouped_gateup_nt", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="host-core time budget of the CPU baseline sample")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-vendor-loop", action="store_true",
                    help="skip timing the per-group torch.matmul (hipBLASLt) loop over the same operands")
    ap.add_argument("--zeros", action="store_true",
                    help="M-grouped bf16 workloads only: all-zero operands (diagnostic: shows how far the clock is held down "
                         "by the power the multipliers draw on random data); reported as data=synthetic-zeros")
    ap.add_argument("--num-cu", type=int, default=-1,
                    help="M-grouped bf16 workloads only: cap the persistent grid at this many workgroups (diagnostic)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (reference kernel for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the grouped-GEMM path has no cross-GPU step; run with --gpus 1", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path)", file=sys.stderr)
        return 2
    from triton_grouped_gemm_amd import _native
    _native.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if (args.zeros or args.num_cu > 0) and WORKLOADS[args.workload][0] != "mg":
        print("--zeros / --num-cu apply to the bf16_m_grouped_* workloads only", file=sys.stderr)
        return 2
    fn, flops, nbytes, dtype_tag, config, cpu_sample = build_workload(args.workload, dev, zeros=args.zeros, num_cu=args.num_cu)
    if args.num_cu > 0:
        config["num_cu"] = args.num_cu

    if args.copy_calibration:
        src = torch.empty(1 << 28, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        fn()
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream(dev)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for s, e in evs:
        s.record(stream)
        fn()
        e.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kernel_ms = [s.elapsed_time(e) for s, e in evs]
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)

    is_gemm = flops > 0
    traffic = MEASURED_TRAFFIC_GB.get(args.workload)
    traffic = None if traffic is None else round(traffic * 1e9)  # bytes per launch
    if is_gemm:
        value = flops / (wall_ms * 1e-3) / 1e12
        peak = PEAK_TFLOPS["fp8" if dtype_tag == "fp8" else "bf16"]
        achieved = flops / (avg_kernel_ms * 1e-3) / 1e12
        roofline = dict(bound="mfma", achieved=round(achieved, 2), peak=peak, unit="TFLOP/s",
                        frac=round(achieved / peak, 4), traffic=traffic,
                        min_ms=round(min(kernel_ms), 4), avg_ms=round(avg_kernel_ms, 4),
                        algorithmic_gbytes=round(nbytes / 1e9, 3))
        metric, unit = "grouped GEMM TFLOP/s (2*M*N*K/time), M-grouped G=128", "TFLOP/s"
    else:
        value = nbytes / (wall_ms * 1e-3) / 1e9
        achieved = nbytes / (avg_kernel_ms * 1e-3) / 1e9
        roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                        frac=round(achieved / PEAK_HBM_GBS, 4), traffic=traffic,
                        min_ms=round(min(kernel_ms), 4), avg_ms=round(avg_kernel_ms, 4))
        metric, unit = "streaming kernel algorithmic GB/s", "GB/s"

    vendor = None
    if build_workload.vendor_loop is not None and not args.no_vendor_loop:
        vl = build_workload.vendor_loop
        vl()
        torch.cuda.synchronize()
        n_v = 3
        tv = time.perf_counter()
        for _ in range(n_v):
            vl()
        torch.cuda.synchronize()
        v_ms = (time.perf_counter() - tv) * 1e3 / n_v
        vendor = dict(value=round(flops / (v_ms * 1e-3) / 1e12, 2), unit="TFLOP/s", ms_per_step=round(v_ms, 4),
                      kind="torch.matmul per group (hipBLASLt), same operands, wall time incl. launches")

    cpu_baseline = None
    if cpu_sample is not None and not args.no_cpu_baseline:
        tf, sample = cpu_sample(args.cpu_seconds)
        cpu_baseline = dict(value=round(tf, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                            sample=sample, host_cpus=os.cpu_count())

    print(json.dumps({
        "metric": metric, "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype_tag, "data": "synthetic-zeros" if args.zeros else "synthetic", "config": config,
        "roofline": roofline, "cpu_baseline": cpu_baseline, "vendor_loop": vendor,
    }))
    return 0


if __name__ == "__main__":
    sys.exit(main())

#!/usr/bin/env python3
"""Headline benchmark: BF16 M-grouped GEMM, G=128, M=655360, N=1536, K=2048 on one MI355X.

One "step" is one pass of the hot path (one ``m_grouped_gemm`` launch) over a synthetic batch whose
operands are already resident in HBM.  Prints ONE JSON line: TFLOP/s = 2*M*N*K / time, the MFMA
roofline fraction of the GEMM kernel (HIP-event timed on the launch stream) and, beside it, the
reference's per-group torch matmul timed on this box's host cores over a bounded sample of groups.

With no flags the same run also times the FP8 block-scaled M-grouped configuration (the other half of the
headline metric, under the "fp8" key of the line, with its own CPU baseline) and the other configurations of the
path, each with its roofline: "masked" (decode-style masked GEMM: the HBM roof binds, the MFMA figure sits beside
it), "k_grouped" (weight gradient), "quant_trans128" (transposing 128x128 quantizer) and "quant_token128" (1x128
activation quantizer).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--dtype bf16|fp16]
                  [--uniform-groups | --random-groups [--unaligned-random-groups] [--group-align 64]]
                  [--no-cpu-baseline] [--no-extras]
  python bench.py --reference-cases [--only-model 30B|235B] [--groups 128] [--active 10] [--warmup 5] [--seed 2026]
                  [--dtype bf16|fp16] [--random-groups ...] [--skip-check] [--skip-vendor] [--csv out.csv]
      the sixteen cases of the reference's own benchmark main (gemm/BF16/m_grouped_gemm_TMA.py:474-493, :602-800),
      with its flags, its group-size draws, its correctness gate and its CSV columns; prints its per-case lines.
"""
from __future__ import annotations

import argparse
import csv
import hashlib
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
# Each figure belongs to the kernel sources it was measured with: name -> (GB, source set).  `roofline.traffic` is
# printed only while the hash of that source set still equals the stamp below; after any change to those files it
# is null until the counters are read again (python bench.py --print-traffic-stamps prints the current hashes).
MEASURED_TRAFFIC_GB = {
    "bf16_m_grouped_gateup_nt": (11.27, "gemm16"),
    "bf16_m_grouped_gateup_nn": (10.11, "gemm16"),
    "bf16_m_grouped_gateup_fp8_out": (10.77, "gemm16"),
    "bf16_m_grouped_down_nt": (5.27, "gemm16"),
    "bf16_m_grouped_down_nn": (5.37, "gemm16"),
    "bf16_masked_decode": (2.47, "gemm16"),
    "bf16_k_grouped_wgrad": (27.75, "gemm16"),
    "fp8_block_m_grouped": (25.36, "gemm8"),
    "fp8_channel_m_grouped": (26.46, "gemm8"),
    "fp8_channel_k_grouped": (16.63, "gemm8"),
    "quant_trans128": (8.12, "quant"),
    "quant_token128": (8.2, "quant"),
    "moe_permute": (3.06, "permute"),      # the row mover (the sort kernels move < 1 % of that)
    "moe_unpermute": (3.07, "permute"),
}
TRAFFIC_SOURCES = {
    "gemm16": ("common.hpp", "sched.hpp", "fast_common.hpp", "gemm_fast.hip", "gemm_w4.hip"),
    "gemm8": ("common.hpp", "sched.hpp", "fast_common.hpp", "gemm_fp8.hip"),
    "quant": ("common.hpp", "sched.hpp", "quant.hip"),
    "permute": ("moe_permute.hip",),
}
TRAFFIC_STAMPS = {  # sha256 over the source set's files, first 16 hex digits, at the time of the counter runs
    "gemm16": "50d017604463b3db",
    "gemm8": "cbf27bfcd62a9ad0",
    "quant": "fdeb1a17e16eb1db",
    "permute": "0231abd86ff30831",
}


def source_stamp(source_set: str) -> str:
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES[source_set]:
        with open(os.path.join(ROOT, "triton_grouped_gemm_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(name: str):
    """Bytes per launch from the table above, or None when there is no figure for this workload or the kernel
    sources have changed since it was measured."""
    entry = MEASURED_TRAFFIC_GB.get(name)
    if entry is None:
        return None
    gb, source_set = entry
    try:
        return round(gb * 1e9) if source_stamp(source_set) == TRAFFIC_STAMPS[source_set] else None
    except OSError:
        return None

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
    # The other shapes of the reference's published tables (README.md:99-140: 16 M-grouped and 8 K-grouped cases on
    # 128 uniform groups of 5120 rows -- run these with --uniform-groups to sit beside them) ...
    "bf16_m_grouped_235b_gateup_nt": ("mg", 3072, 4096, True),
    "bf16_m_grouped_235b_gateup_nn": ("mg", 3072, 4096, False),
    "bf16_m_grouped_235b_down_nt": ("mg", 4096, 1536, True),
    "bf16_m_grouped_235b_down_nn": ("mg", 4096, 1536, False),
    "bf16_k_grouped_30b_gateup": ("kg", 2048, 1536, False),
    "bf16_k_grouped_30b_down": ("kg", 768, 2048, False),
    "bf16_k_grouped_235b_down": ("kg", 1536, 4096, False),
    # ... and its two FP8 examples (README.md:168-169; gemm/FP8/m_grouped_gemm_channel_expert.py:293-308,
    # gemm/FP8/k_grouped_gemm_channel_expert.py:276-296): 32 experts with fixed token counts, activations e5m2,
    # weights e4m3fn; the K-grouped one with every expert's tokens padded to a multiple of 128.
    "fp8_channel_m_grouped_readme": ("fp8c", 6144, 5120, True, dict(sizes=[509, 3587, 125, 3971] * 8, fmt_a="e5m2")),
    "fp8_channel_k_grouped_readme": ("fp8ck", 6144, 5120, False, dict(sizes=[512, 3584, 128, 3968] * 8, fmt_a="e5m2")),
    # the headline's shape as ONE dense GEMM through the vendor library (torch.matmul -> hipBLASLt): the whole A against
    # one expert's weights.  Not a grouped GEMM: the yardstick for what this silicon gives a dense kernel on this shape.
    "vendor_dense_gateup": ("dense", 1536, 2048, True),
    "quant_trans128": ("quant", 4096, 0, False),
    "quant_token128": ("quant1", 0, 4096, False),    # the 1x128 activation quantizer on [M, K] bf16
    # MoE token movement either side of the GEMMs: 81920 tokens x top-8 = 655360 rows of 2048 bf16
    "moe_permute": ("permute", 2048, 8, False),       # hidden, topK
    "moe_unpermute": ("unpermute", 2048, 8, False),
}


METRICS = {
    "mg": "grouped GEMM TFLOP/s (2*M*N*K/time), BF16 M-grouped G=128",
    "mgq": "grouped GEMM TFLOP/s (2*M*N*K/time), BF16 M-grouped G=128, output quantised 1x128 in the epilogue",
    "masked": "grouped GEMM TFLOP/s (2*valid_rows*N*K/time), BF16 masked M-grouped G=128",
    "kg": "grouped GEMM TFLOP/s (2*K_total*M*N/time), BF16 K-grouped G=128",
    "fp8": "grouped GEMM TFLOP/s (2*M*N*K/time), FP8 block-scaled M-grouped G=128",
    "fp8c": "grouped GEMM TFLOP/s (2*M*N*K/time), FP8 per-channel M-grouped G=128",
    "fp8ck": "grouped GEMM TFLOP/s (2*K_total*M*N/time), FP8 per-channel K-grouped G=128",
    "dense": "vendor library dense GEMM TFLOP/s (2*M*N*K/time), torch.matmul on the headline's shape",
    "quant": "transposing 128x128 quantizer, algorithmic GB/s",
    "quant1": "1x128 activation quantizer (per_token_cast_to_fp8), algorithmic GB/s",
    "permute": "MoE permute (sort + row mover), algorithmic GB/s",
    "unpermute": "MoE unpermute, algorithmic GB/s",
}


def build_workload(name: str, dev, seed: int = 2026, zeros: bool = False, num_cu: int = -1, uniform: bool = False,
                   groups: int = None, m_total: int = None, dtype: str = "bf16", size_mode: str = None,
                   group_align: int = 64):
    """Returns (fn, flops_per_step, algorithmic_bytes_per_step, dtype_tag, description, cpu_sample_fn); leaves a
    per-group library-GEMM loop over the same operands in ``build_workload.vendor_loop`` where one exists, the
    tensor that loop writes in ``build_workload.vendor_out`` and the operands in ``build_workload.operands``.
    ``uniform``: every group gets m_total / groups rows (the reference's published tables use 128 groups of 5120
    rows) instead of the Dirichlet-multinomial draw.  ``size_mode`` "random" / "random-unaligned": the draws of the
    reference's benchmark main for --random-groups (blocks of ``group_align`` rows) / --unaligned-random-groups.
    ``dtype`` "fp16": 16-bit GEMM workloads on half precision operands.  ``groups`` / ``m_total`` shrink the
    problem (tests)."""
    build_workload.vendor_loop = None
    build_workload.vendor_dense = None
    build_workload.vendor_out = None
    build_workload.vendor_kind = None
    build_workload.operands = {}
    from triton_grouped_gemm_amd import workloads as wl
    from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import m_grouped_gemm
    kind, N, K, trans_b, *extra = WORKLOADS[name]
    opts = extra[0] if extra else {}
    G = groups or globals()["G"]
    M_TOTAL = m_total or globals()["M_TOTAL"]
    if "sizes" in opts and not groups:  # the workload states its own group sizes
        sizes_cpu = torch.tensor(opts["sizes"], dtype=torch.int32)
        G, M_TOTAL = len(opts["sizes"]), int(sum(opts["sizes"]))
        size_tag = "as the reference's example: " + " ".join(map(str, opts["sizes"][:4])) + f" x {G // 4}"
    elif size_mode in ("random", "random-unaligned"):
        sizes_cpu = wl.reference_group_sizes(G, M_TOTAL, seed, False, group_align, size_mode == "random")
        size_tag = (f"random as the reference's --random-groups, blocks of {group_align} rows" if size_mode == "random"
                    else "random as the reference's --unaligned-random-groups (exact sum, no alignment)")
    else:
        sizes_cpu = wl.uniform_sizes(G, M_TOTAL) if uniform else wl.dirichlet_multinomial_sizes(G, M_TOTAL, 128, seed=seed)
        size_tag = f"uniform, {M_TOTAL // G} rows per group" if uniform else "dirichlet-multinomial, 128-aligned"
    sizes = sizes_cpu.to(dev)
    t16 = torch.float16 if dtype == "fp16" else torch.bfloat16
    tag16 = "fp16" if dtype == "fp16" else "bf16"

    def randn16(shape, scale, sd):  # N(0,1)*scale in the 16-bit type of the run (fp16: the bf16 draw, converted)
        x = wl.randn_bf16(shape, scale, sd, dev)
        return x if t16 == torch.bfloat16 else x.to(t16)
    fp8_a = torch.float8_e5m2 if opts.get("fmt_a") == "e5m2" else torch.float8_e4m3fn
    bounds = [(int(s0), int(s0 + n)) for s0, n in zip((sizes_cpu.cumsum(0) - sizes_cpu).tolist(), sizes_cpu.tolist())]
    if kind == "mg":
        a = randn16((M_TOTAL, K), K ** -0.5, seed + 1)
        b = randn16((G, N, K) if trans_b else (G, K, N), K ** -0.5, seed + 2)
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
            return done_flops / t_used / 1e12, f"{groups} largest groups of {G} ({done_flops / flops * 100:.1f}% of the step's flops), {tag16} torch matmul per group"
        c_ref = torch.empty((M_TOTAL, N), device=dev, dtype=t16)

        def vendor_loop():  # one library GEMM per expert, the GPU baseline the reference's tables compare against
            for g, (s0, s1) in enumerate(bounds):
                if s1 > s0:
                    torch.matmul(a[s0:s1], b[g].t() if trans_b else b[g], out=c_ref[s0:s1])
        build_workload.vendor_loop = vendor_loop
        build_workload.vendor_out = c_ref
        # the same shape as one dense GEMM: the whole A against the first expert's weights
        build_workload.vendor_dense = lambda: torch.matmul(a, b[0].t() if trans_b else b[0], out=c_ref)
        return fn, flops, nbytes, tag16, dict(workload=name, G=G, M=M_TOTAL, N=N, K=K, trans_b=trans_b,
                                              group_sizes=size_tag, seed=seed), cpu_sample
    if kind == "dense":
        a = randn16((M_TOTAL, K), K ** -0.5, seed + 1)
        w = randn16((N, K), K ** -0.5, seed + 2)
        if zeros:
            a.zero_()
            w.zero_()
        c = torch.empty((M_TOTAL, N), device=dev, dtype=t16)
        fn = lambda: torch.matmul(a, w.t(), out=c)
        return (fn, 2.0 * M_TOTAL * N * K, 2.0 * M_TOTAL * K + 2.0 * N * K + 2.0 * M_TOTAL * N, tag16,
                dict(workload=name, M=M_TOTAL, N=N, K=K, kernel="torch.matmul (hipBLASLt), one dense GEMM", seed=seed), None)
    if kind == "mgq":
        from triton_grouped_gemm_amd.gemm.fused import m_grouped_gemm_fp8_out
        a = wl.randn_bf16((M_TOTAL, K), K ** -0.5, seed + 1, dev)
        b = wl.randn_bf16((G, N, K), K ** -0.5, seed + 2, dev)
        fn = lambda: m_grouped_gemm_fp8_out(a, b, sizes, trans_b, scales_mn_major=True)
        nbytes = 2.0 * M_TOTAL * K + 2.0 * G * N * K + 1.0 * M_TOTAL * N + 4.0 * M_TOTAL * N / 128
        return (fn, 2.0 * M_TOTAL * N * K, nbytes, "bf16",
                dict(workload=name, G=G, M=M_TOTAL, N=N, K=K, trans_b=trans_b, output="e4m3fn codes + 1x128 fp32 scales",
                     group_sizes=size_tag, seed=seed), None)
    if kind == "masked":
        from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_masked_TMA import m_grouped_gemm_masked
        m_max = 512
        mm_cpu = wl.masked_counts(G, m_max, seed)
        mm = mm_cpu.to(dev)
        lhs = randn16((G * m_max, K), K ** -0.5, seed + 1)
        rhs = randn16((G, N, K), K ** -0.5, seed + 2)
        out = torch.empty((G * m_max, N), device=dev, dtype=t16)
        mv = float(mm_cpu.sum())
        fn = lambda: m_grouped_gemm_masked(lhs, rhs, out, mm, m_max)
        return (fn, 2.0 * mv * N * K, 2.0 * mv * K + 2.0 * int((mm_cpu > 0).sum()) * N * K + 2.0 * mv * N, tag16,
                dict(workload=name, G=G, m_max=m_max, N=N, K=K, valid_rows=int(mv), seed=seed), None)
    if kind == "kg":
        from triton_grouped_gemm_amd.gemm.BF16.k_grouped_gemm_TMA import k_grouped_gemm
        Nd, Md = N, K
        a = randn16((M_TOTAL, Md), 1.0, seed + 1)
        b = randn16((M_TOTAL, Nd), 1.0, seed + 2)
        fn = lambda: k_grouped_gemm(a, b, sizes)
        c_ref = torch.zeros((G, Md, Nd), device=dev, dtype=t16)

        def vendor_loop():
            for g, (s0, s1) in enumerate(bounds):
                if s1 > s0:
                    torch.matmul(a[s0:s1].t(), b[s0:s1], out=c_ref[g])
        build_workload.vendor_loop = vendor_loop
        build_workload.vendor_out = c_ref
        return (fn, 2.0 * M_TOTAL * Md * Nd, 2.0 * M_TOTAL * (Md + Nd) + 2.0 * G * Md * Nd, tag16,
                dict(workload=name, G=G, K_total=M_TOTAL, M_dim=Md, N_dim=Nd, group_sizes=size_tag, seed=seed), None)
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
        build_workload.operands = dict(aq=aq, wq=wq, out=out, sizes=sizes)
        c_ref = torch.empty((M_TOTAL, N), device=dev, dtype=torch.bfloat16)
        one = torch.ones((), device=dev, dtype=torch.float32)

        def vendor_loop():  # one library FP8 GEMM per expert on the same codes; it applies NO block scales
            for g, (s0, s1) in enumerate(bounds):
                if s1 > s0:
                    c_ref[s0:s1] = torch._scaled_mm(aq[0][s0:s1], wq[0][g].t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
        build_workload.vendor_loop = vendor_loop
        build_workload.vendor_out = c_ref
        build_workload.vendor_kind = "torch._scaled_mm per group (hipBLASLt), same fp8 codes, unit scales: no block scaling"
        flops = 2.0 * M_TOTAL * N * K

        def cpu_sample(budget_s: float):
            """The oracle's computation for this path on the host cores: dequantise both operands (1x128 and 128x128
            scales), fp32 matmul, group by group, largest groups first until the time budget is used."""
            from oracle import gemm_ref
            order = torch.argsort(sizes_cpu, descending=True).tolist()
            done_flops, t_used, n_groups = 0.0, 0.0, 0
            for g in order:
                s0, s1 = bounds[g]
                if s1 == s0:
                    continue
                ag, sg = aq[0][s0:s1].float().cpu(), aq[1][s0:s1].cpu().contiguous()
                wg, wsg = wq[0][g:g + 1].float().cpu(), wq[1][g:g + 1].cpu()
                if n_groups == 0:  # thread pool and allocator warm-up on a few rows
                    gemm_ref.fp8_block_scaled_reference(ag[:128], sg[:128], wg, wsg, [128])
                t0 = time.perf_counter()
                gemm_ref.fp8_block_scaled_reference(ag, sg, wg, wsg, [s1 - s0])
                t_used += time.perf_counter() - t0
                done_flops += 2.0 * (s1 - s0) * N * K
                n_groups += 1
                if t_used >= budget_s:
                    break
            return done_flops / t_used / 1e12, (f"{n_groups} largest groups of {G} ({done_flops / flops * 100:.1f}% of the step's flops), "
                                                "dequantise + fp32 torch matmul per group")
        return (fn, flops, nbytes, "fp8",
                dict(workload=name, G=G, M=M_TOTAL, N=N, K=K, recipe="1x128 act / 128x128 weight, e4m3fn",
                     group_sizes=size_tag, seed=seed), cpu_sample)
    if kind == "fp8c":
        from triton_grouped_gemm_amd.gemm.FP8.m_grouped_gemm_channel_expert import gmm_fp8_act_per_channel_w_per_expert
        gen = torch.Generator(device=dev).manual_seed(seed + 3)
        a = wl.randn_bf16((M_TOTAL, K), 1.0, seed + 1, dev).to(fp8_a)
        w = wl.randn_bf16((G, N, K), 1.0, seed + 2, dev).to(torch.float8_e4m3fn)
        sa = torch.rand(M_TOTAL, 1, device=dev, generator=gen) + 0.5
        sb = torch.rand(G * N, device=dev, generator=gen) + 0.5
        fn = lambda: gmm_fp8_act_per_channel_w_per_expert(a, sa, w, sb, sizes, torch.bfloat16)
        nbytes = M_TOTAL * K + 4.0 * M_TOTAL + G * N * K + 4.0 * G * N + 2.0 * M_TOTAL * N
        build_workload.operands = dict(a=a, sa=sa, w=w, sb=sb, sizes=sizes)
        c_ref = torch.empty((M_TOTAL, N), device=dev, dtype=torch.bfloat16)
        sb_rows = sb.view(G, 1, N)

        def vendor_loop():  # one library FP8 GEMM per expert with row-wise scales: the same arithmetic
            for g, (s0, s1) in enumerate(bounds):
                if s1 > s0:
                    c_ref[s0:s1] = torch._scaled_mm(a[s0:s1], w[g].t(), scale_a=sa[s0:s1], scale_b=sb_rows[g], out_dtype=torch.bfloat16)
        build_workload.vendor_loop = vendor_loop
        build_workload.vendor_out = c_ref
        build_workload.vendor_kind = "torch._scaled_mm per group (hipBLASLt), row-wise scales, same operands"
        return (fn, 2.0 * M_TOTAL * N * K, nbytes, "fp8",
                dict(workload=name, G=G, M=M_TOTAL, N=N, K=K,
                     recipe="per-token x per-channel scales, " + ("e5m2 x e4m3fn" if fp8_a == torch.float8_e5m2 else "e4m3fn"),
                     group_sizes=size_tag, seed=seed), None)
    if kind == "fp8ck":
        from triton_grouped_gemm_amd.gemm.FP8.k_grouped_gemm_channel_expert import matmul as k_grouped_fp8
        m_dim, n_dim = K, N
        gen = torch.Generator(device=dev).manual_seed(seed + 3)
        x = wl.randn_bf16((m_dim, M_TOTAL), 1.0, seed + 1, dev).to(fp8_a)
        y = wl.randn_bf16((n_dim, M_TOTAL), 1.0, seed + 2, dev).to(torch.float8_e4m3fn)
        xs = torch.rand(m_dim, G, device=dev, generator=gen) + 0.5
        ys = torch.rand(n_dim, G, device=dev, generator=gen) + 0.5
        code_a = 2 if fp8_a == torch.float8_e5m2 else 1
        fn = lambda: k_grouped_fp8(x, xs, y, ys, sizes, m_dim, n_dim, M_TOTAL, G, dtype_a=code_a, dtype_b=1)
        nbytes = 1.0 * M_TOTAL * (m_dim + n_dim) + 4.0 * G * (m_dim + n_dim) + 2.0 * G * m_dim * n_dim
        return (fn, 2.0 * M_TOTAL * m_dim * n_dim, nbytes, "fp8",
                dict(workload=name, G=G, M=m_dim, N=n_dim, K_total=M_TOTAL,
                     recipe="per-channel x per-expert scales, " + ("e5m2 x e4m3fn" if code_a == 2 else "e4m3fn"),
                     group_sizes=size_tag, seed=seed), None)
    if kind == "quant":
        from triton_grouped_gemm_amd.quant.trans_per_block_quant_expand_128x import trans_per_block_quant_expand_128x
        x = wl.randn_bf16((M_TOTAL, N), 1.0, seed + 1, dev)
        me = M_TOTAL + 128 * G - M_TOTAL % 128
        fn = lambda: trans_per_block_quant_expand_128x(x, sizes)
        nbytes = 2.0 * M_TOTAL * N + 1.0 * N * me + 4.0 * (N / 128) * (me / 128)
        return fn, 0.0, nbytes, "bf16->fp8", dict(workload=name, G=G, M=M_TOTAL, N=N, seed=seed), None
    if kind == "quant1":
        from triton_grouped_gemm_amd.quant.fp8_cast import per_token_cast_to_fp8
        x = wl.randn_bf16((M_TOTAL, K), 1.0, seed + 1, dev)
        fn = lambda: per_token_cast_to_fp8(x, scales_mn_major=True)
        nbytes = 2.0 * M_TOTAL * K + 1.0 * M_TOTAL * K + 4.0 * M_TOTAL * K / 128
        return fn, 0.0, nbytes, "bf16->fp8", dict(workload=name, M=M_TOTAL, K=K, scales="[K/128, M]", seed=seed), None
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


MIN_WARM_MS = 150.0   # the clocks of a chip that has been idle settle over roughly 100 ms of work
MIN_TIMED_MS = 60.0
SHORT_STEP_MS = 1.5


def time_workload(fn, steps: int, warmup: int, dev, stretch: bool = False):
    """`warmup` untimed launches, then `steps` launches each bracketed by HIP events on the launch stream.
    A workload whose step takes well under a millisecond would spend the whole measurement on a chip that is still
    raising its clocks (masked decode: 0.555 ms per step after 12 warm-up launches, 0.525 after 300, same box), so the
    warm-up of a step shorter than SHORT_STEP_MS goes on until MIN_WARM_MS of launches have been issued (steps of
    several milliseconds measure the same either way: the requested count stands); with ``stretch`` (the secondary
    workloads of the default line) the timed region of such a workload grows to at least MIN_TIMED_MS as well.
    Returns (wall ms per step, list of per-launch event times in ms, launches timed, warm-up launches done)."""
    t0 = time.perf_counter()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    done = warmup
    step_ms = (time.perf_counter() - t0) * 1e3 / max(warmup, 1)
    if warmup > 0 and step_ms < SHORT_STEP_MS and step_ms * warmup < MIN_WARM_MS:
        more = min(2000, int(MIN_WARM_MS / max(step_ms, 1e-3)) + 1 - warmup)
        for _ in range(more):
            fn()
        torch.cuda.synchronize()
        done += more
        if stretch:
            steps = max(steps, min(2000, int(MIN_TIMED_MS / max(step_ms, 1e-3)) + 1))
    stream = torch.cuda.current_stream(dev)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for s, e in evs:
        s.record(stream)
        fn()
        e.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return wall_ms, [s.elapsed_time(e) for s, e in evs], steps, done


def summarise(name: str, flops: float, nbytes: float, dtype_tag: str, wall_ms: float, kernel_ms, default_draw: bool):
    """(value, unit, roofline dict) of one timed workload.  ``default_draw``: the workload ran on the group sizes and
    data type the traffic counters were read on (the Dirichlet draw, bf16): only then is the measured traffic its."""
    avg_kernel_ms = sum(kernel_ms) / len(kernel_ms)
    traffic = measured_traffic(name) if default_draw else None  # bytes per launch, or None
    if flops > 0:
        value = flops / (wall_ms * 1e-3) / 1e12
        peak = PEAK_TFLOPS["fp8" if dtype_tag == "fp8" else "bf16"]
        achieved = flops / (avg_kernel_ms * 1e-3) / 1e12
        roofline = dict(bound="mfma", achieved=round(achieved, 2), peak=peak, unit="TFLOP/s",
                        frac=round(achieved / peak, 4), traffic=traffic,
                        min_ms=round(min(kernel_ms), 4), avg_ms=round(avg_kernel_ms, 4),
                        algorithmic_gbytes=round(nbytes / 1e9, 3))
        if WORKLOADS[name][0] == "masked":
            # Decode-style masked GEMM: about 200 flop per algorithmic byte, below the ridge (312 for bf16), so the HBM
            # roof is the one that binds.  It is the roofline of the line; the MFMA figure goes beside it.
            gbs = nbytes / (avg_kernel_ms * 1e-3) / 1e9
            hbm = dict(bound="hbm", achieved=round(gbs, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                       frac=round(gbs / PEAK_HBM_GBS, 4), traffic=traffic,
                       min_ms=round(min(kernel_ms), 4), avg_ms=round(avg_kernel_ms, 4),
                       algorithmic_gbytes=round(nbytes / 1e9, 3), mfma=roofline)
            return value, "TFLOP/s", hbm
        return value, "TFLOP/s", roofline
    value = nbytes / (wall_ms * 1e-3) / 1e9
    achieved = nbytes / (avg_kernel_ms * 1e-3) / 1e9
    roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                    frac=round(achieved / PEAK_HBM_GBS, 4), traffic=traffic,
                    min_ms=round(min(kernel_ms), 4), avg_ms=round(avg_kernel_ms, 4))
    return value, "GB/s", roofline


def time_vendor_dense(flops: float, steps: int, warmup: int, dev):
    """The workload's shape as one dense vendor-library GEMM (left behind by build_workload for the M-grouped 16-bit
    workloads), event-timed like the library's own launches; None where there is none."""
    vd = getattr(build_workload, "vendor_dense", None)
    if vd is None:
        return None
    _, kms, _, _ = time_workload(vd, steps, warmup, dev)
    avg = sum(kms) / len(kms)
    return dict(value=round(flops / (avg * 1e-3) / 1e12, 2), unit="TFLOP/s", avg_ms=round(avg, 4), min_ms=round(min(kms), 4),
                kind="torch.matmul (hipBLASLt): the whole A against one expert's weights, i.e. the same M x N x K as ONE dense GEMM")


def time_vendor_loop(flops: float):
    """The per-group library-GEMM loop that build_workload left behind, or None (also when the library refuses the call)."""
    vl = build_workload.vendor_loop
    if vl is None:
        return None
    try:
        vl()
        torch.cuda.synchronize()
        n_v = 3
        tv = time.perf_counter()
        for _ in range(n_v):
            vl()
        torch.cuda.synchronize()
    except Exception as exc:  # e.g. a scaling mode this torch / hipBLASLt build does not offer
        return dict(value=None, unit="TFLOP/s", kind=getattr(build_workload, "vendor_kind", ""), error=str(exc).splitlines()[0][:200])
    v_ms = (time.perf_counter() - tv) * 1e3 / n_v
    kind = getattr(build_workload, "vendor_kind", None) or "torch.matmul per group (hipBLASLt), same operands"
    return dict(value=round(flops / (v_ms * 1e-3) / 1e12, 2), unit="TFLOP/s", ms_per_step=round(v_ms, 4),
                kind=kind + ", wall time incl. launches")


REFERENCE_CASES = [  # the reference's BENCHMARK_CASES (gemm/BF16/m_grouped_gemm_TMA.py:474-493): model, n, k, total_m, trans_b
    ("30B", 1536, 2048, 655360, True), ("30B", 1536, 2048, 655360, True),
    ("30B", 1536, 2048, 655360, False), ("30B", 1536, 2048, 655360, False),
    ("30B", 2048, 768, 655360, True), ("30B", 2048, 768, 655360, True),
    ("30B", 2048, 768, 655360, False), ("30B", 2048, 768, 655360, False),
    ("235B", 3072, 4096, 655360, True), ("235B", 3072, 4096, 655360, True),
    ("235B", 3072, 4096, 655360, False), ("235B", 3072, 4096, 655360, False),
    ("235B", 4096, 1536, 655360, True), ("235B", 4096, 1536, 655360, True),
    ("235B", 4096, 1536, 655360, False), ("235B", 4096, 1536, 655360, False),
]


def event_min_avg(fn, warmup: int, active: int):
    """The reference's ``benchmark_cuda_event`` (gemm/BF16/m_grouped_gemm_TMA.py:584-599): ``warmup`` untimed calls,
    then ``active`` calls each between two events; (min ms, mean ms)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(active):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        fn()
        e.record()
        e.synchronize()
        times.append(s.elapsed_time(e))
    return min(times), sum(times) / len(times)


def run_reference_cases(args, dev) -> int:
    """The reference's benchmark main, case by case, on this library: same cases, flags, group-size draws, operands
    (unscaled torch.randn), timing and correctness gate (row-max normalisation, assert_close at 1e-2 against the
    per-group torch matmul); the per-group library GEMM loop stands where its cuBLAS extension stood."""
    from oracle import gemm_ref
    from triton_grouped_gemm_amd import workloads as wl
    from triton_grouped_gemm_amd.gemm.BF16.m_grouped_gemm_TMA import _build_m_grouped_metadata, _m_grouped_gemm_launch
    torch.manual_seed(args.seed)
    torch.cuda.manual_seed_all(args.seed)
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float16
    cases = [c for c in REFERENCE_CASES if args.only_model is None or c[0] == args.only_model]
    results = []
    for case_idx, (model, n, k, total_m, trans_b) in enumerate(cases):
        torch.cuda.empty_cache()
        sizes_cpu = wl.reference_group_sizes(args.groups, total_m, args.seed + case_idx, not args.random_groups,
                                             args.group_align, not args.unaligned_random_groups)
        sizes = sizes_cpu.to(device=dev, dtype=torch.int64)
        M = int(sizes_cpu.sum())
        assert M == total_m, f"generated M={M}, expected {total_m}"
        starts = sizes_cpu.to(torch.int64).cumsum(0) - sizes_cpu
        bad_8, bad_64 = int((starts % 8 != 0).sum()), int((starts % 64 != 0).sum())
        metadata = _build_m_grouped_metadata(sizes)
        a = torch.randn(M, k, dtype=dtype, device=dev)
        b = torch.randn((args.groups, n, k) if trans_b else (args.groups, k, n), dtype=dtype, device=dev)
        layout = "B[G,N,K]" if trans_b else "B[G,K,N]"
        out = torch.empty(M, n, dtype=dtype, device=dev)
        lib_min, lib_avg = event_min_avg(lambda: _m_grouped_gemm_launch(a, b, out, sizes, trans_b, args.num_sm, metadata=metadata),
                                         args.warmup, args.active)
        bounds = [(int(s0), int(s0 + c)) for s0, c in zip(starts.tolist(), sizes_cpu.tolist())]
        v_min = v_avg = 0.0
        if not args.skip_vendor:
            c_ref = torch.empty_like(out)

            def vendor():
                for g, (s0, s1) in enumerate(bounds):
                    if s1 > s0:
                        torch.matmul(a[s0:s1], b[g].t() if trans_b else b[g], out=c_ref[s0:s1])
            v_min, v_avg = event_min_avg(vendor, args.warmup, args.active)
            del c_ref
        if not args.skip_check:  # the reference's gate: m_grouped_reference on the same device, row-max normalised, 1e-2
            ref = torch.cat([a[s0:s1] @ (b[g].t() if trans_b else b[g]) for g, (s0, s1) in enumerate(bounds) if s1 > s0])
            torch.testing.assert_close(gemm_ref.row_max_normalization(out.float()), gemm_ref.row_max_normalization(ref.float()),
                                       rtol=1e-2, atol=1e-2)
            del ref
        flops = 2.0 * M * n * k
        print(f"[{case_idx:02d}] model={model}, n={n}, k={k}, M={M}, trans_b={trans_b}, layout={layout}, out_layout=C[M,N], "
              f"bad_start_align8={bad_8}/{args.groups}, bad_start_align64={bad_64}/{args.groups}", flush=True)
        print(f"    HIP kernel GPU time {lib_min:.2f} ms min / {lib_avg:.2f} ms avg, {flops / lib_min / 1e9:.0f} TFLOP/s min-time / "
              f"{flops / lib_avg / 1e9:.0f} TFLOP/s avg-time", flush=True)
        if v_min > 0:
            print(f"    hipBLASLt per-group loop GPU time {v_min:.2f} ms min / {v_avg:.2f} ms avg, {flops / v_min / 1e9:.0f} TFLOP/s; "
                  f"speedup {v_min / lib_min:.2f}x (baseline_layout={layout})", flush=True)
        results.append({
            "case_idx": case_idx, "model": model, "n": n, "k": k, "M": M, "trans_b": trans_b, "layout": layout,
            "output_layout": "C[M,N]", "groups": args.groups, "dtype": args.dtype,
            "kernel_min_ms": lib_min, "kernel_avg_ms": lib_avg,
            "kernel_tflops_min_time": flops / lib_min / 1e9, "kernel_tflops_avg_time": flops / lib_avg / 1e9,
            "vendor_loop_min_ms": v_min, "vendor_loop_avg_ms": v_avg,
            "vendor_loop_tflops_min_time": flops / v_min / 1e9 if v_min > 0 else 0.0,
            "speedup_vs_vendor_loop": v_min / lib_min if v_min > 0 else 0.0,
            "group_sizes": "uniform" if not args.random_groups else ("random-unaligned" if args.unaligned_random_groups else f"random-align{args.group_align}"),
            "bad_start_align8": bad_8, "bad_start_align64": bad_64,
        })
        del a, b, out
    if args.csv:
        os.makedirs(os.path.dirname(os.path.abspath(args.csv)), exist_ok=True)
        with open(args.csv, "w", newline="") as f:
            writer = csv.DictWriter(f, fieldnames=list(results[0].keys()))
            writer.writeheader()
            writer.writerows(results)
        print(f"Wrote CSV summary to {args.csv}", flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed launches first (default 12: the first ten or so run at a clock that is still settling, "
                         "4.2 -> 3.3 ms on the headline; --reference-cases: 5, as the reference)")
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="default: bf16_m_grouped_gateup_nt, followed by the other configurations of the path under their own keys")
    ap.add_argument("--dtype", choices=["bf16", "fp16"], default="bf16", help="16-bit GEMM workloads: operand and output type")
    group_mode = ap.add_mutually_exclusive_group()
    group_mode.add_argument("--uniform-groups", action="store_true",
                            help="every group gets M / G = 5120 rows, as in the reference's published tables, instead of the "
                                 "Dirichlet-multinomial draw (the default of --reference-cases, as in the reference)")
    group_mode.add_argument("--random-groups", action="store_true",
                            help="group sizes as the reference's --random-groups draws them, in blocks of --group-align rows")
    ap.add_argument("--unaligned-random-groups", action="store_true",
                    help="with --random-groups: exact-sum random sizes without alignment")
    ap.add_argument("--group-align", type=int, default=64, help="alignment, in rows, of --random-groups sizes")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="host-core time budget of each CPU baseline sample")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-vendor-loop", action="store_true",
                    help="skip timing the per-group library GEMM loop (hipBLASLt through torch) over the same operands")
    ap.add_argument("--no-fp8", action="store_true", help="default run: skip the FP8 block-scaled half")
    ap.add_argument("--no-extras", action="store_true",
                    help="default run: skip the masked, K-grouped and quantizer configurations that follow the two headline halves")
    ap.add_argument("--zeros", action="store_true",
                    help="M-grouped bf16 workloads only: all-zero operands (diagnostic: shows how far the clock is held down "
                         "by the power the multipliers draw on random data); reported as data=synthetic-zeros")
    ap.add_argument("--num-cu", type=int, default=-1,
                    help="M-grouped bf16 workloads only: cap the persistent grid at this many workgroups (diagnostic)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (reference kernel for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--print-traffic-stamps", action="store_true",
                    help="print the current hashes of the kernel source sets that the measured-traffic table is stamped with")
    # the reference's benchmark main (gemm/BF16/m_grouped_gemm_TMA.py:602-635), flag for flag
    ap.add_argument("--reference-cases", action="store_true", help="run the reference's sixteen M-grouped cases and print its per-case lines")
    ap.add_argument("--groups", type=int, default=128)
    ap.add_argument("--active", type=int, default=10, help="--reference-cases: timed launches per case")
    ap.add_argument("--seed", type=int, default=2026)
    ap.add_argument("--num-sm", type=int, default=-1, help="--reference-cases: cap on the persistent grid (numSM)")
    ap.add_argument("--skip-check", action="store_true", help="--reference-cases: skip the correctness gate")
    ap.add_argument("--skip-vendor", "--skip-cublas", dest="skip_vendor", action="store_true",
                    help="--reference-cases: skip the per-group library GEMM loop (the reference's --skip-cublas)")
    ap.add_argument("--csv", type=str, default="", help="--reference-cases: write the summary as CSV")
    ap.add_argument("--only-model", choices=["30B", "235B"], default=None)
    args = ap.parse_args()
    if args.print_traffic_stamps:
        print(json.dumps({k: source_stamp(k) for k in TRAFFIC_SOURCES}))
        return 0
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the grouped-GEMM path has no cross-GPU step; run with --gpus 1", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path)", file=sys.stderr)
        return 2
    if args.unaligned_random_groups and not args.random_groups:
        print("--unaligned-random-groups goes with --random-groups", file=sys.stderr)
        return 2
    from triton_grouped_gemm_amd import _native
    _native.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.reference_cases:
        args.warmup = 5 if args.warmup is None else args.warmup
        return run_reference_cases(args, dev)
    args.warmup = 12 if args.warmup is None else args.warmup
    workload = args.workload or "bf16_m_grouped_gateup_nt"
    default_run = args.workload is None and not args.zeros and args.num_cu <= 0
    with_fp8 = default_run and not args.no_fp8
    with_extras = default_run and not args.no_extras
    kind = WORKLOADS[workload][0]
    if (args.zeros and kind not in ("mg", "dense")) or (args.num_cu > 0 and kind != "mg"):
        print("--zeros applies to the bf16_m_grouped_* and vendor_dense_* workloads, --num-cu to bf16_m_grouped_* only", file=sys.stderr)
        return 2
    if (args.uniform_groups or args.random_groups) and kind in ("masked", "quant", "quant1", "permute", "unpermute"):
        print("--uniform-groups / --random-groups apply to the M-grouped and K-grouped GEMM workloads", file=sys.stderr)
        return 2
    if args.dtype != "bf16" and kind not in ("mg", "masked", "kg", "dense"):
        print("--dtype fp16 applies to the 16-bit M-grouped, masked and K-grouped GEMM workloads", file=sys.stderr)
        return 2
    size_mode = None if not args.random_groups else ("random-unaligned" if args.unaligned_random_groups else "random")
    default_draw = not (args.uniform_groups or args.random_groups) and args.dtype == "bf16" and args.groups == 128
    groups = None if args.groups == 128 else args.groups

    def build(name):
        return build_workload(name, dev, seed=args.seed, zeros=args.zeros and name == workload, num_cu=args.num_cu,
                              uniform=args.uniform_groups, groups=groups, dtype=args.dtype, size_mode=size_mode,
                              group_align=args.group_align)

    def cpu_base(sample_fn):
        if sample_fn is None or args.no_cpu_baseline:
            return None
        tf, sample = sample_fn(args.cpu_seconds)
        return dict(value=round(tf, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port", sample=sample,
                    host_cpus=os.cpu_count())

    fn, flops, nbytes, dtype_tag, config, cpu_sample = build(workload)
    if args.num_cu > 0:
        config["num_cu"] = args.num_cu

    if args.copy_calibration:
        src = torch.empty(1 << 28, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    wall_ms, kernel_ms, steps_done, warm_done = time_workload(fn, args.steps, args.warmup, dev)
    value, unit, roofline = summarise(workload, flops, nbytes, dtype_tag, wall_ms, kernel_ms, default_draw)
    vendor = None if args.no_vendor_loop else time_vendor_loop(flops)
    vendor_dense = None if args.no_vendor_loop else time_vendor_dense(flops, args.steps, args.warmup, dev)
    cpu_baseline = cpu_base(cpu_sample)

    line = {
        "metric": METRICS[kind].replace("G=128", f"G={config['G']}") if "G" in config else METRICS[kind], "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": steps_done,
        "warmup": warm_done, "ms_per_step": round(wall_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype_tag, "data": "synthetic-zeros" if args.zeros else "synthetic", "config": config,
        "roofline": roofline, "cpu_baseline": cpu_baseline, "vendor_loop": vendor,
    }
    if vendor_dense is not None:
        line["vendor_dense"] = vendor_dense

    def release():
        build_workload.vendor_loop = build_workload.vendor_out = build_workload.vendor_dense = None
        build_workload.operands = {}
        torch.cuda.empty_cache()

    if with_fp8:  # the FP8 half of the headline metric: same run, same steps and warm-up, its own operands
        del fn, cpu_sample
        release()
        name8 = "fp8_block_m_grouped"
        fn8, flops8, nbytes8, tag8, config8, cpu8 = build(name8)
        wall8, kms8, _, _ = time_workload(fn8, args.steps, args.warmup, dev)
        value8, unit8, roof8 = summarise(name8, flops8, nbytes8, tag8, wall8, kms8, default_draw)
        line["fp8"] = {"metric": METRICS["fp8"], "value": round(value8, 2), "unit": unit8, "ms_per_step": round(wall8, 4),
                       "dtype": tag8, "config": config8, "roofline": roof8,
                       "vendor_loop": None if args.no_vendor_loop else time_vendor_loop(flops8),
                       "cpu_baseline": cpu_base(cpu8)}
        del fn8, cpu8
    if with_extras:  # the other configurations of the path, each with its roofline
        for key, name in (("masked", "bf16_masked_decode"), ("k_grouped", "bf16_k_grouped_wgrad"),
                          ("quant_trans128", "quant_trans128"), ("quant_token128", "quant_token128")):
            release()
            fnx, flopsx, nbytesx, tagx, configx, _ = build(name)
            wallx, kmsx, stepsx, warmx = time_workload(fnx, args.steps, args.warmup, dev, stretch=True)
            valuex, unitx, roofx = summarise(name, flopsx, nbytesx, tagx, wallx, kmsx, default_draw)
            line[key] = {"metric": METRICS[WORKLOADS[name][0]], "value": round(valuex, 2), "unit": unitx,
                         "steps": stepsx, "warmup": warmx, "ms_per_step": round(wallx, 4), "dtype": tagx, "config": configx,
                         "roofline": roofx}
            del fnx
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

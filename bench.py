#!/usr/bin/env python3
"""Benchmark of the Pairformer hot path on one MI355X.

One "step" is one full Pairformer block (triangle multiplication out/in,
triangle attention start/end, pair transition, pair-biased single attention,
single transition) at N_token = 768, c_pair = 128, c_single = 384, bf16 residual
stream, synthetic N(0,1) inputs resident in HBM, random-init weights N(0,0.02),
last 10% of the tokens masked as padding.  Prints ONE JSON line:

  metric / value   Pairformer ms per block (lower is better)
  roofline         the dominant kernel (by time per block) against the MI355X
                   dense bf16 MFMA peak, its launch timed live with HIP events on
                   all-ones masks (nothing skipped); `padded` inside it: the same
                   launch under the workload's padding
  cpu_baseline     the CPU oracle (eager PyTorch restatement of the reference
                   formulas, fp32) timed on this host's cores on a bounded
                   sample, scaled to the metric's unit
  per_op_ms / tflops_per_op   informational breakdown

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--n-token N]
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0
PROFILES = os.path.join(ROOT, "profiles")


def measured_traffic_bytes(kernel, n):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 counter summary of this workload
    (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, the factors from a plain elementwise kernel of known size
    in the same profiler run, see --calibrate): column `total MB` of
    profiles/pairformer_block_n<N>_bf16_hbm_traffic.txt.  None when there is no summary for this size."""
    try:
        with open(os.path.join(PROFILES, f"pairformer_block_n{n}_bf16_hbm_traffic.txt")) as f:
            for line in f:
                cols = line.split()
                if len(cols) == 7 and cols[0] == kernel:
                    return float(cols[5]) * 1e6
    except (OSError, ValueError):
        pass
    return None


def kernel_time_shares(n, top=6):
    """Per-kernel share of the GPU time of one block at N_token = n from the committed kernel-trace
    summary profiles/pairformer_block_n<N>_bf16_kernel_stats.txt: {kernel: [avg us per launch, % of time]}."""
    shares = {}
    try:
        with open(os.path.join(PROFILES, f"pairformer_block_n{n}_bf16_kernel_stats.txt")) as f:
            for line in f:
                cols = line.split()
                if len(cols) >= 6 and "_kernel" in cols[0] and cols[-1].replace(".", "", 1).isdigit():
                    try:
                        shares[cols[0].split("<")[0]] = [float(cols[-4]), float(cols[-1])]
                    except ValueError:
                        continue
    except OSError:
        return None
    return dict(sorted(shares.items(), key=lambda kv: -kv[1][1])[:top]) or None


def flops_trimul(n):      # one direction
    return 256.0 * n ** 3 + 196608.0 * n ** 2


def flops_triattn(n):     # one direction
    return 512.0 * n ** 3 + 164864.0 * n ** 2


def flops_block(n):
    return (2 * flops_trimul(n) + 2 * flops_triattn(n) + 393216.0 * n ** 2
            + 5632.0 * n ** 2 + 1474560.0 * n + 3538944.0 * n)


def flops_contraction(n):     # the N x N x N contraction of 128 channels alone
    return 256.0 * n ** 3


def flops_attention_core(n):  # QK^T and PV for N rows x 4 heads x d=32
    return 512.0 * n ** 3


def random_init_(module, gen, std=0.02):
    """Random-init weights for timing: every matrix and bias N(0, std), every
    LayerNorm weight (and the other 1-D `weight` vectors) 1 + N(0, std).  Only
    bench.py's cpu_baseline leg touches the CPU oracle; the timed modules get
    their parameters here."""
    import torch
    with torch.no_grad():
        for name, p in module.named_parameters():
            noise = torch.randn(p.shape, generator=gen) * std
            if p.dim() == 1 and name.endswith("weight"):
                noise += 1.0
            p.copy_(noise)
    if hasattr(module, "invalidate"):
        module.invalidate()
    return module


def gpu_time_ms(fn, iters, warmup=2, warm_ms=0.0):
    """Average duration of fn() in ms, timed with HIP events on torch's current
    stream (the stream handed to the C ABI).  `warm_ms`: keep launching untimed
    until that much wall time has passed (after an idle stretch the GPU clock
    takes some tens of milliseconds to come back to its sustained level)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < warm_ms:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _timed(fn, max_iters, budget_s):
    """1 warm-up + up to `max_iters` timed calls (fewer when `budget_s` runs out; at
    least one), wall clock: the method of the reference's own kernel tests
    (kernel_test/triangle_multiplication.py:192-231).  Returns (mean_s, min_s, iterations)."""
    t0 = time.perf_counter()
    fn()
    warm = time.perf_counter() - t0
    times = []
    spent = warm
    while len(times) < max_iters and (not times or spent + times[-1] <= budget_s):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
        spent += times[-1]
    return sum(times) / len(times), min(times), len(times)


def cpu_baseline(n_metric):
    """The CPU oracle (this build's eager-PyTorch restatement of the reference
    formulas; the reference's own xfold + libxsmm path cannot be built here) on
    this host's cores, on a bounded sample: one Pairformer block at N=384 in fp32
    and in torch.bfloat16 with all threads, and the 4-block N=128 fp32 stack with
    all threads and with one.  `value` is the fp32 N=384 mean scaled by algorithmic
    FLOPs to the metric's N (flagged as extrapolated)."""
    import torch
    from oracle import af3_oracle as O
    g = torch.Generator().manual_seed(0)
    threads = torch.get_num_threads()
    affinity = len(os.sched_getaffinity(0))

    def block_case(n, dtype, nblocks=1):
        blocks = [O.cast_params(O.make_pairformer_block_params(g), dtype) for _ in range(nblocks)]
        pair = torch.randn(n, n, 128, generator=g).to(dtype)
        single = torch.randn(n, 384, generator=g).to(dtype)
        seq = (torch.arange(n) < (int(0.9 * n) if nblocks == 1 else n)).to(dtype)
        pm = seq[:, None] * seq[None, :]

        def run():
            with torch.no_grad():
                O.pairformer_stack(pair, pm, single, seq, blocks)
        return run

    legs = {}
    n_cpu = 384
    mean, mn, it = _timed(block_case(n_cpu, torch.float32), 10, 14.0)
    legs["block_n384_fp32"] = {"mean_ms": round(mean * 1e3, 1), "min_ms": round(mn * 1e3, 1), "iterations": it,
                               "threads": threads}
    fp32_mean = mean
    mean, mn, it = _timed(block_case(n_cpu, torch.bfloat16), 10, 8.0)
    legs["block_n384_bf16"] = {"mean_ms": round(mean * 1e3, 1), "min_ms": round(mn * 1e3, 1), "iterations": it,
                               "threads": threads}
    mean, mn, it = _timed(block_case(128, torch.float32, 4), 10, 5.0)
    legs["stack4_n128_fp32"] = {"mean_ms": round(mean * 1e3, 1), "min_ms": round(mn * 1e3, 1), "iterations": it,
                                "threads": threads}
    torch.set_num_threads(1)
    try:
        mean, mn, it = _timed(block_case(128, torch.float32, 4), 10, 6.0)
    finally:
        torch.set_num_threads(threads)
    legs["stack4_n128_fp32_1thread"] = {"mean_ms": round(mean * 1e3, 1), "min_ms": round(mn * 1e3, 1),
                                        "iterations": it, "threads": 1}
    scaled_ms = fp32_mean * 1e3 * flops_block(n_metric) / flops_block(n_cpu)
    return {
        "value": round(scaled_ms, 1), "unit": "ms/block", "cores": threads, "kind": "port",
        "extrapolated": n_metric != n_cpu,
        "sample": (f"CPU oracle (eager PyTorch restatement of the reference formulas; not xfold+TPP, which cannot be "
                   f"built here), 1 warm-up + up to 10 timed runs each, wall clock: one Pairformer block at "
                   f"N={n_cpu} (10% padded) fp32 and bf16, the 4-block N=128 fp32 stack with all threads and with "
                   f"one; value = fp32 N={n_cpu} mean ({fp32_mean * 1e3:.0f} ms on {threads} threads) scaled by "
                   f"algorithmic FLOPs to N={n_metric} (extrapolated)"),
        "legs": legs, "torch_threads": threads, "sched_affinity": affinity, "cpu_model": _cpu_model(),
    }


def diffusion_step(pkg, n, dev, samples=5, iters=20):
    """One denoising evaluation of the diffusion head (atom cross-attention
    encoder, 24-block diffusion transformer, decoder) on `samples` samples of an
    n-token synthetic batch with 24 atom slots per token, bf16 activations,
    random-init weights; the per-batch conditioning is computed once, as the
    sampler does, and timed separately."""
    import torch
    g = torch.Generator().manual_seed(1)
    head = random_init_(pkg.nn.DiffusionHead(), g).to(dev)
    head.load_hip_params()
    batch = pkg.nn.atom_layout.synthetic_batch(n, g, n_padding_tokens=n // 10).to(dev)
    emb = {"single": torch.randn(n, 384, generator=g).to(dev), "pair": torch.randn(n, n, 128, generator=g).to(dev),
           "target_feat": torch.randn(n, 447, generator=g).to(dev)}
    sampler = pkg.nn.DiffusionSampler(head, num_samples=samples)
    _, t_hat, _ = sampler.schedule(dev)

    def setup():
        sc, pc = head.pre_conditioning(batch, emb, t_hat, True)
        return sc, pc, head.prepare(batch, emb, pc)
    setup()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    sc, pc, state = setup()
    torch.cuda.synchronize()
    setup_ms = (time.perf_counter() - t0) * 1e3
    pos = torch.randn(samples, n, 24, 3, generator=g).to(dev) * float(t_hat[100])
    ms = gpu_time_ms(lambda: head(pos, t_hat[100], batch, emb, sc[100], pc, state=state), iters, warm_ms=40.0)
    ms_ref = gpu_time_ms(lambda: head(pos, t_hat[100], batch, emb, sc[100], pc), 5)
    return {"workload": f"one denoising evaluation, {samples} samples, N_token={n}, 24 atom slots per token, "
                        "24 transformer blocks, 3+3 atom-attention blocks, bf16 activations",
            "ms_per_evaluation": round(ms, 3),
            "ms_per_evaluation_conditioning_recomputed": round(ms_ref, 3),
            "per_batch_setup_ms": round(setup_ms, 1),
            "sampling_200_steps_s": round((setup_ms + 200 * ms) / 1e3, 3)}


def evoformer_block_ms(pkg, n, dev, rows=1024, iters=10):
    """One Evoformer (MSA) block: outer-product mean, MSA pair-weighted
    averaging, MSA transition and the five pair operators, bf16 streams."""
    import torch
    g = torch.Generator().manual_seed(2)
    blk = random_init_(pkg.nn.EvoformerBlock(), g).to(dev)
    blk.load_hip_params()
    msa = torch.randn(rows, n, 64, generator=g).to(dev).bfloat16()
    pair = torch.randn(n, n, 128, generator=g).to(dev).bfloat16()
    seq = (torch.arange(n) < int(0.9 * n)).float().to(dev)
    mm = seq[None, :].expand(rows, n).contiguous()
    pm = (seq[:, None] * seq[None, :]).contiguous()
    ms = gpu_time_ms(lambda: blk(msa, pair, mm, pm), iters, warm_ms=40.0)
    ms_opm = gpu_time_ms(lambda: blk.outer_product_mean.run(msa, mm, residual=pair), iters)
    ms_att = gpu_time_ms(lambda: blk.msa_attention1.run(msa, mm, pair, residual=True), iters)
    flops_opm = 2.0 * (32 * n) ** 2 * rows + 2.0 * n * n * 1024 * 128
    return {"workload": f"one Evoformer block, {rows} MSA rows x {n} tokens, c_msa=64, c_pair=128, bf16",
            "ms_per_block": round(ms, 3), "outer_product_mean_ms": round(ms_opm, 3),
            "outer_product_mean_tflops": round(flops_opm / ms_opm / 1e9, 1), "msa_attention_ms": round(ms_att, 3)}


def template_block_ms(pkg, n, dev, iters=10):
    """The Pairformer block of the template embedding (nn/d_template.py:198-201): 64 pair channels, transition
    factor 2, no single track.  It runs on the 128-channel kernels over zero-padded operands."""
    import torch
    g = torch.Generator().manual_seed(5)
    blk = random_init_(pkg.nn.PairformerBlock(c_pair=64, num_intermediate_factor=2, with_single=False), g).to(dev)
    blk.load_hip_params()
    pair = torch.randn(n, n, 64, generator=g).to(dev).bfloat16()
    seq = (torch.arange(n) < int(0.9 * n)).float().to(dev)
    pm = (seq[:, None] * seq[None, :]).contiguous()
    ms = gpu_time_ms(lambda: blk(pair, pm), iters, warm_ms=40.0)
    return {"workload": f"one Pairformer block on 64 pair channels (template embedding), N_token={n}, bf16, "
                        "10% trailing tokens masked, padded to the 128-channel kernels",
            "ms_per_block": round(ms, 3)}


def trunk_recycle_ms(pkg, n, dev, rows=1024, iters=3):
    """One recycling pass of the Evoformer trunk: input embeddings, 4 Evoformer
    (MSA) blocks, 48 Pairformer blocks (no template embedding), bf16 streams."""
    import torch
    g = torch.Generator().manual_seed(3)
    mod = random_init_(pkg.nn.Evoformer(), g).to(dev)
    mod.load_hip_params()
    batch = pkg.nn.atom_layout.synthetic_trunk_batch(n, rows, g, n_padding_tokens=n // 10).to(dev)
    tf = torch.randn(n, 447, generator=g).to(dev)
    prev = {"pair": torch.randn(n, n, 128, generator=g).to(dev), "single": torch.randn(n, 384, generator=g).to(dev)}
    ms = gpu_time_ms(lambda: mod(batch, prev, tf), iters, warmup=1)
    return {"workload": f"one recycling pass of the trunk: embeddings + 4 Evoformer blocks ({rows} MSA rows) + 48 "
                        f"Pairformer blocks, N_token={n}, bf16",
            "ms_per_recycle": round(ms, 2)}


def trunk_n1536(pkg, dev, n=1536, blocks=48, passes=2):
    """The 48 Pairformer blocks of the trunk (distinct random weights) on one
    resident [1536, 1536, 128] bf16 pair tensor, all-ones masks and 10% trailing
    padding: wall time of a whole pass through PairformerStack, host-timed
    around a device synchronisation."""
    import torch
    g = torch.Generator().manual_seed(4)
    stack = random_init_(pkg.nn.PairformerStack(num_blocks=blocks), g).to(dev)
    stack.load_hip_params()
    pair0 = torch.randn(n, n, 128, generator=g).bfloat16().to(dev)
    single0 = torch.randn(n, 384, generator=g).bfloat16().to(dev)
    res = {"workload": f"{blocks}-block Pairformer trunk, N_token={n}, c_pair=128, c_single=384, bf16 residual "
                       "stream, distinct random-init weights per block, whole pair tensor resident on one GPU",
           "blocks": blocks}
    for label, live in (("unmasked", n), ("padded_10pct", int(0.9 * n))):
        sm = (torch.arange(n) < live).float().to(dev)
        pm = (sm[:, None] * sm[None, :]).contiguous()
        best = None
        for i in range(passes + 1):                      # the first pass is the warm-up
            pair, single = pair0.clone(), single0.clone()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            pair, single = stack(pair, pm, single, sm)
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3
            if i > 0:
                best = ms if best is None else min(best, ms)
        if not torch.isfinite(pair.float()).all():
            raise RuntimeError("non-finite pair activations after the trunk")
        res[label] = {"ms_total": round(best, 2), "ms_per_block": round(best / blocks, 3),
                      "tflops": round(blocks * flops_block(n) / best / 1e9, 1)}
    # where a block's time goes at this size: [avg us per launch, % of GPU time] from the committed summary
    res["per_kernel_share"] = kernel_time_shares(n)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--n-token", type=int, default=768)
    ap.add_argument("--io", choices=["bf16", "f32"], default="bf16", help="dtype of the residual stream")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--all-ones", action="store_true",
                    help="all-ones masks for every leg (no padding), for profiles of the roofline launch")
    ap.add_argument("--no-trunk", action="store_true", help="skip the 48-block N=1536 trunk timing")
    ap.add_argument("--no-diffusion", action="store_true",
                    help="skip the diffusion-head, Evoformer-block and 64-channel-block timings")
    ap.add_argument("--only", choices=["diffusion-head", "evoformer-block", "trunk-recycle"],
                    help="run that leg alone and print its object (for profiler runs)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run a plain elementwise kernel that reads and writes 256 MiB, three times: the "
                         "reference against which the FETCH_SIZE / WRITE_SIZE counters of a profiler run are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build keeps the whole pair tensor on ONE GPU (no sharding, no collectives); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import __graft_entry__ as ge
    pkg = ge.load_package()
    pkg.lib.load()                       # raises if the HIP library is missing

    dev = torch.device("cuda:0")
    n = args.n_token
    if args.only:
        leg = {"diffusion-head": diffusion_step, "evoformer-block": evoformer_block_ms,
               "trunk-recycle": trunk_recycle_ms}[args.only](pkg, n, dev)
        print(json.dumps({args.only: leg}))
        return
    io = torch.bfloat16 if args.io == "bf16" else torch.float32
    g = torch.Generator().manual_seed(0)
    blk = random_init_(pkg.nn.PairformerBlock(), g).to(dev)
    blk.load_hip_params()
    pair = torch.randn(n, n, 128, generator=g).to(dev).to(io)
    single = torch.randn(n, 384, generator=g).to(dev).to(io)
    live = int(0.9 * n)

    def masks(live_tokens):
        sm = (torch.arange(n) < live_tokens).float().to(dev)
        return sm, (sm[:, None] * sm[None, :]).contiguous()

    seq_mask, pair_mask = masks(live)
    seq_ones, pair_ones = masks(n)

    # A step is one Pairformer block.  The timed steps run back to back the way the trunk runs its 48
    # blocks (nn.pairformer_loop): block i's update of `single`, a chain of small kernels, goes on a second
    # stream beside block i + 1's pair operators.  Everything launched is waited for before the clock stops.
    # `isolated` is the same block called on its own, one stream, per call.
    loop = pkg.nn.pairformer_loop

    def timed(pm, sm):
        loop([blk] * args.warmup, pair, pm, single, sm)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        loop([blk] * args.steps, pair, pm, single, sm)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        if not torch.isfinite(pair.float()).all():
            raise RuntimeError("non-finite pair activations after the timed steps")
        pair.normal_(generator=None)
        single.normal_(generator=None)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            blk(pair, pm, single, sm)
        torch.cuda.synchronize()
        iso = (time.perf_counter() - t0) * 1e3 / args.steps
        pair.normal_(generator=None)
        single.normal_(generator=None)
        return ms, iso

    if args.all_ones:   # (for profiles: every launch of the run then does all of the algorithm's work)
        seq_mask, pair_mask, live = seq_ones, pair_ones, n
    ms_per_step, ms_isolated = timed(pair_mask, seq_mask)
    # the same block with nothing masked: every kernel leaves out work on padding (fully masked prologue tiles,
    # rows without a live key, key tiles without one), so the padded figure flatters the kernels by that much
    ms_unmasked, ms_unmasked_isolated = timed(pair_ones, seq_ones)

    # ---- per-operator breakdown (untimed with respect to the headline) ----
    it = max(3, min(args.steps, 10))

    def per_op_times(pm):
        t = {
            "trimul_out": gpu_time_ms(lambda: blk.triangle_multiplication_outgoing.run(pair, pm, True), it),
            "trimul_in": gpu_time_ms(lambda: blk.triangle_multiplication_incoming.run(pair, pm, True), it),
            "triattn_start": gpu_time_ms(lambda: blk.pair_attention1.run(pair, pm, True), it),
            "triattn_end": gpu_time_ms(lambda: blk.pair_attention2.run(pair, pm, True), it),
            "pair_transition": gpu_time_ms(lambda: blk.pair_transition.run(pair, True), it),
        }
        fl = {"trimul_out": flops_trimul(n), "trimul_in": flops_trimul(n), "triattn_start": flops_triattn(n),
              "triattn_end": flops_triattn(n), "pair_transition": 393216.0 * n * n}
        return t, {k: fl[k] / t[k] / 1e9 for k in t}

    per_op, tflops_per_op = per_op_times(pair_mask)
    per_op_un, tflops_per_op_un = per_op_times(pair_ones)

    # ---- roofline of the dominant kernel, one launch timed with HIP events ----
    npad = (n + 7) // 8 * 8
    a = (torch.randn(128, n, npad, generator=g) * 0.1).to(dev).bfloat16()
    b = (torch.randn(128, n, npad, generator=g) * 0.1).to(dev).bfloat16()
    a[:, :, n:] = 0
    b[:, :, n:] = 0
    t_buf = torch.empty_like(a)
    q_, k_ = ((torch.randn(n, 4, n, 32, generator=g) * 0.5).to(dev).bfloat16() for _ in range(2))
    vt_ = pkg.ops.pack_vt((torch.randn(n, 4, 32, n, generator=g) * 0.5).to(dev).bfloat16())
    nb = pkg.ops.pack_pair_bias(torch.randn(4, n, n, generator=g).to(dev))
    og = torch.empty((n * n, 128), dtype=torch.bfloat16, device=dev)
    # (the operands above are generated on the host, during which the GPU idles and its clock drops)
    ms_contract = gpu_time_ms(lambda: pkg.ops.triangle_contraction(a, b, t_buf), 30, warm_ms=40.0)
    ms_attn = gpu_time_ms(lambda: pkg.ops.grid_attention_core(q_, k_, vt_, nb, pair_mask, og), 30, warm_ms=40.0)
    ms_attn_un = gpu_time_ms(lambda: pkg.ops.grid_attention_core(q_, k_, vt_, nb, pair_ones, og), 30,
                             warm_ms=40.0)
    # FLOPs the attention core executes under the trailing padding: a row without a live key takes the uniform
    # shortcut (no products), a live row visits only the 64-key tiles that hold a live key, all N queries each
    executed_attn = 512.0 * live * n * (64.0 * ((live + 63) // 64))

    # The roofline object is on the ALL-ONES mask: the kernel then executes exactly the algorithm's FLOPs, so
    # the fraction is neither flattered by skipped padding nor dependent on how the padding falls on tiles.
    # `padded` beside it is the same launch under the workload's 10 % padding, on both counts of FLOPs.
    kernels = {
        "contract_kernel (triangle contraction)": (ms_contract, flops_contraction(n)),
        "triattn_flash_kernel (triangle attention core)": (ms_attn_un, flops_attention_core(n)),
    }
    dom = max(kernels, key=lambda k: kernels[k][0])      # each runs twice per block
    dom_ms, dom_flops = kernels[dom]
    achieved = dom_flops / dom_ms / 1e9
    roofline = {
        "kernel": dom, "mask": "all-ones (nothing skipped: algorithmic FLOPs = executed FLOPs)",
        "bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
        "unit": "TFLOP/s", "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
        "traffic": measured_traffic_bytes(dom.split(" ")[0], n),
        "launch_ms": round(dom_ms, 4),
        "others": {k: {"launch_ms": round(v[0], 4), "tflops": round(v[1] / v[0] / 1e9, 2),
                       "frac": round(v[1] / v[0] / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)}
                   for k, v in kernels.items() if k != dom},
    }
    if dom.startswith("triattn") and not args.all_ones:
        roofline["padded"] = {
            "mask": "10% trailing tokens masked (the workload of `value`)",
            "launch_ms": round(ms_attn, 4),
            "frac_algorithmic_flops": round(flops_attention_core(n) / ms_attn / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
            "frac_executed_flops": round(executed_attn / ms_attn / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
            "executed_share_of_algorithmic_flops": round(executed_attn / flops_attention_core(n), 4),
        }
    del a, b, t_buf, q_, k_, vt_, nb, og

    # ---- the target run: the 48-block trunk at 1536 tokens, whole pair tensor resident ----
    trunk = None if args.no_trunk else trunk_n1536(pkg, dev)

    # ---- the diffusion head that calls the diffusion transformer / atom cross-attention (informational) ----
    diffusion = None
    if not args.no_diffusion:
        diffusion = diffusion_step(pkg, n, dev)
    evo = None if args.no_diffusion else evoformer_block_ms(pkg, n, dev)
    template = None if args.no_diffusion else template_block_ms(pkg, n, dev)

    if args.calibrate:
        cx = torch.zeros(64 * 1024 * 1024, dtype=torch.float32, device=dev)   # 256 MiB in, 256 MiB out
        cy = torch.empty_like(cx)
        for _ in range(3):
            torch.add(cx, 1.0, out=cy)
        torch.cuda.synchronize()
        del cx, cy

    out = {
        "metric": "Pairformer ms/block at N=%d bf16" % n,
        "value": round(ms_per_step, 4), "unit": "ms/block", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"one Pairformer block, N_token={n}, c_pair=128, c_single=384, "
                               f"{args.io} residual stream, bf16 MFMA operands / fp32 accumulate, "
                               "10% trailing tokens masked, random-init weights N(0,0.02); steps run back to "
                               "back as the trunk loop runs its blocks (single update of one block on a second "
                               "stream beside the pair operators of the next)"},
        "isolated_block_ms": round(ms_isolated, 4),
        "block_tflops": round(flops_block(n) / ms_per_step / 1e9, 2),
        "per_op_ms": {k: round(v, 4) for k, v in per_op.items()},
        "tflops_per_op": {k: round(v, 2) for k, v in tflops_per_op.items()},
        "roofline": roofline,
        "unmasked": {
            "workload": "the same block with all-ones masks (no padding: nothing is skipped)",
            "value": round(ms_unmasked, 4), "unit": "ms/block",
            "isolated_block_ms": round(ms_unmasked_isolated, 4),
            "block_tflops": round(flops_block(n) / ms_unmasked / 1e9, 2),
            "per_op_ms": {k: round(v, 4) for k, v in per_op_un.items()},
            "tflops_per_op": {k: round(v, 2) for k, v in tflops_per_op_un.items()},
        },
    }
    if trunk is not None:
        out["trunk_n1536"] = trunk
    if diffusion is not None:
        out["diffusion_head"] = diffusion
    if template is not None:
        out["template_block_c64"] = template
    if evo is not None:
        out["evoformer_block"] = evo
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(n)
    print(json.dumps(out))


if __name__ == "__main__":
    main()

"""Benchmark of the retention hot path on one MI355X.

A step is one forward + backward of fused_chunk_retention over one synthetic batch of
benchmark configuration 2 (bf16, B=8 H=16 T=4096 dk=dv=128, zero initial state, dO ~ N(0,1)), inputs
resident in HBM.  Prints ONE JSON line: whole-job TFLOP/s from the algorithmic FLOP count
(dense chunk-64 tiles, no recompute), tokens/s, the HBM roofline of the backward kernel (the
dominant launch of a step) measured with events on the launch stream, the same step timed from
an idle device, the other benchmark configurations each with a roofline object of its own, and
the CPU oracle timed on the host cores beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--spin-up S] [--no-cpu] [--no-pop] [--no-long]
                    [--no-layer5] [--no-layer] [--no-model]
    python bench.py --profile-leg {headline,pop_fused,pop_two_op,long,layer5,layer_ops} --steps K
        exactly K steps of one workload and nothing else: what the rocprofv3 runs of profile_counters.sh trace
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "flash-pop_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)
TESTS = os.path.join(ROOT, "tests")     # the model harness and (CPU leg only) the oracle's helpers live there

CHUNK = 64
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0
SPIN_UP_SECONDS = 0.3        # see spin_up()


def profiled_traffic(kernel):
    """HBM bytes per launch of `kernel` at config 2 as the hardware counters gave them (FETCH_SIZE and
    WRITE_SIZE, each scaled by what it reads for a plain copy of known size).  The figure is not
    measured by this script: it is read from the summary under profiles/ that the counter runs
    of profile_counters.sh produced, together with the commit it was measured at.
    -> (bytes or None, commit or None)"""
    return _profile_line(r"^HBM_TRAFFIC %s(?:<[^>]*>)? bytes_per_launch=(\d+) measured_at=(\w+)", kernel)


def profiled_step_traffic(leg):
    """HBM bytes per step of a whole workload (all its launches), from the same counter runs:
    `HBM_TRAFFIC_STEP <leg> bytes_per_step=<n> measured_at=<commit>`.  -> (bytes or None, commit or None)"""
    return _profile_line(r"^HBM_TRAFFIC_STEP %s bytes_per_step=(\d+) measured_at=(\w+)", leg)


def _profile_line(pattern, name):
    import glob
    import re
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        with open(path) as f:
            m = re.search(pattern % re.escape(name), f.read(), re.M)
        if m:
            return int(m.group(1)), m.group(2)
    return None, None


def spin_up(step, seconds=SPIN_UP_SECONDS):
    """Part of set-up, before the warm-up steps: keeps the device busy with the benchmarked step
    until its clocks have settled.  From idle the first ~50 steps (~25 ms) of this workload run up
    to 20 % slower than every later one; a run of `--warmup 5 --steps 20` would time only that ramp."""
    import torch
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        n += 10
    return n


def algorithmic_flops(B, T, H, dk, dv, C=CHUNK):
    fwd = 2 * (C * (dk + dv) + 2 * dk * dv)
    bwd = 2 * (C * (3 * dk + 2 * dv) + 4 * dk * dv)
    n = B * T * H
    return fwd * n, bwd * n


def algorithmic_bytes(B, T, H, dk, dv):
    n = B * T * H
    return 2 * (2 * dk + 2 * dv) * n, 2 * (4 * dk + 3 * dv) * n


def head_decays(H):
    """gamma_h = 1 - 2^(-5-h) (flash_pop/retnet.py:70-76), as Python floats."""
    return tuple(1.0 - 2.0 ** (-5.0 - h) for h in range(H))


def make_inputs(B, T, H, dk, dv, seed, state_std=None, device="cpu"):
    """q, k, v ~ N(0,1) in bf16 (k is scaled by dk^-1/2 inside the op), generated on the host so that the
    CPU baseline sees the same bits; state_std None: no state, 0: zeros, else N(0, std^2)."""
    import torch
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, dk, generator=g).to(torch.bfloat16)
    k = torch.randn(B, T, H, dk, generator=g).to(torch.bfloat16)
    v = torch.randn(B, T, H, dv, generator=g).to(torch.bfloat16)
    if state_std is None:
        s = None
    elif state_std == 0:
        s = torch.zeros(B, H, dk, dv, dtype=torch.bfloat16)
    else:
        s = (torch.randn(B, H, dk, dv, generator=g) * state_std).to(torch.bfloat16)
    return tuple(None if t is None else t.to(device) for t in (q, k, v, s))


def make_cotangents(shapes, seed, device="cpu"):
    import torch
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(*s, generator=g).to(torch.bfloat16).to(device) for s in shapes]


# ---- the workloads: each returns step(ev=None) -> None and a description; ev = three events recorded before the
# forward, between forward and backward and after the backward, on the stream the kernels are launched on -----------

def workload_headline(dev):
    """Config 2: plain retention forward + backward, zero initial state (the caller's zeros: no gradient)."""
    import torch
    from flash_pop_amd import fused_chunk_retention
    B, T, H, dk, dv = 8, 4096, 16, 128, 128
    decays = head_decays(H)
    q, k, v, s = make_inputs(B, T, H, dk, dv, seed=0, state_std=0.0, device=dev)
    d_o, = make_cotangents([(B, T, H, dv)], seed=1, device=dev)
    leaves = [t.requires_grad_() for t in (q, k, v)]

    def step(ev=None):
        if ev:
            ev[0].record()
        o, S = fused_chunk_retention(*leaves, s, decays)
        if ev:
            ev[1].record()
        torch.autograd.grad([o], leaves, [d_o])
        if ev:
            ev[2].record()

    b = algorithmic_bytes(B, T, H, dk, dv)
    return step, {"shape": (B, T, H, dk, dv), "tokens": B * T, "bytes": b, "flops": algorithmic_flops(B, T, H, dk, dv)}


def _pop_workload(dev, B, T, H, dk, dv, block, Ls, fused, seeds):
    import torch
    from flash_pop_amd import fused_chunk_retention, flash_pop_retention
    from flash_pop_amd.pop_retention import flash_pop_retention_with_suffixes
    decays = head_decays(H)
    N = T // block
    q, k, v, s = make_inputs(B, T, H, dk, dv, seed=seeds[0], state_std=0.0, device=dev)
    d_o, = make_cotangents([(B, T, H, dv)], seed=seeds[1], device=dev)
    qs, ks, vs, _ = make_inputs(B * (N + 1), Ls, H, dk, dv, seed=seeds[2], device=dev)
    d_os, = make_cotangents([(B * (N + 1), Ls, H, dv)], seed=seeds[3], device=dev)
    leaves = [t.requires_grad_() for t in (q, k, v)]
    sleaves = [t.requires_grad_() for t in (qs, ks, vs)]

    def step(ev=None):
        if ev:
            ev[0].record()
        if fused:   # the suffixes inside the walks: they read the state at their boundary in place
            o, o_s, _ = flash_pop_retention_with_suffixes(*leaves, s, decays, block, *sleaves)
        else:       # the reference's call sequence
            o, states = flash_pop_retention(*leaves, s, decays, block)
            starts = torch.cat((s[:, None], states), dim=1).flatten(0, 1)
            o_s, _ = fused_chunk_retention(*sleaves, starts, decays)
        if ev:
            ev[1].record()
        torch.autograd.grad([o, o_s], leaves + sleaves, [d_o, d_os])
        if ev:
            ev[2].record()

    tok_ctx, tok_sfx = B * T, B * (N + 1) * Ls
    # every token of the context and of the suffixes once per tensor; the states stay on chip in the fused op
    b = algorithmic_bytes(1, tok_ctx + tok_sfx, H, dk, dv)
    return step, {"shape": (B, T, H, dk, dv), "tokens": tok_ctx + tok_sfx, "tokens_context": tok_ctx, "bytes": b}


def workload_pop_fused(dev):
    """Config 4 through flash_pop_retention_with_suffixes: 64-token blocks, 65 suffixes of 16 tokens per sequence."""
    return _pop_workload(dev, 8, 4096, 16, 128, 128, 64, 16, True, (0, 1, 2, 3))


def workload_pop_two_op(dev):
    """Config 4 through flash_pop_retention, torch.cat of the block states and fused_chunk_retention on the suffix batch."""
    return _pop_workload(dev, 8, 4096, 16, 128, 128, 64, 16, False, (0, 1, 2, 3))


def workload_layer5(dev):
    """The retention op of one layer of config 5's model: B=8 T=2048 H=12 dk=64 dv=128, 64-token blocks,
    33 suffixes of 16 tokens per sequence, through flash_pop_retention_with_suffixes."""
    return _pop_workload(dev, 8, 2048, 12, 64, 128, 64, 16, True, (10, 11, 12, 13))


def workload_long(dev):
    """Config 3: B=2 H=8 T=16384 dk=128 dv=256 with a carried state and its gradient.  16 streams cannot fill 256
    compute units, so the op cuts each sequence into segments (fp_retention_*_split)."""
    import torch
    from flash_pop_amd import fused_chunk_retention
    B, T, H, dk, dv = 2, 16384, 8, 128, 256
    decays = head_decays(H)
    q, k, v, s = make_inputs(B, T, H, dk, dv, seed=4, state_std=0.02, device=dev)
    d_o, d_s = make_cotangents([(B, T, H, dv), (B, H, dk, dv)], seed=5, device=dev)
    leaves = [t.requires_grad_() for t in (q, k, v, s)]

    def step(ev=None):
        if ev:
            ev[0].record()
        o, S = fused_chunk_retention(*leaves, decays)
        if ev:
            ev[1].record()
        torch.autograd.grad([o, S], leaves, [d_o, d_s])
        if ev:
            ev[2].record()

    return step, {"shape": (B, T, H, dk, dv), "tokens": B * T, "bytes": algorithmic_bytes(B, T, H, dk, dv),
                  "flops": algorithmic_flops(B, T, H, dk, dv)}


def workload_layer_ops(dev):
    """The two elementwise stages around the op at config 2's tensor shapes: rotary embedding of q and k, per-head
    norm + swish gate forward and backward, one launch each."""
    import torch
    from flash_pop_amd import XPos, gated_group_norm
    B, T, H, d = 8, 4096, 16, 128
    g = torch.Generator(device=dev).manual_seed(7)
    q, k, r, gate, d_out = (torch.randn(B, T, H, d, generator=g, device=dev).to(torch.bfloat16) for _ in range(5))
    gate, d_out = gate.flatten(-2), d_out.flatten(-2)
    xpos = XPos(d)
    rl, gl = r.requires_grad_(), gate.requires_grad_()

    def step(ev=None):
        xpos(q, k, 0)
        out = gated_group_norm(rl, gl, 1e-6)
        torch.autograd.grad(out, [rl, gl], d_out)

    n = q.numel() * 2
    return step, {"shape": (B, T, H, d, d), "tokens": B * T, "bytes": (7 * n, 5 * n)}


WORKLOADS = {"headline": workload_headline, "layer_ops": workload_layer_ops, "pop_fused": workload_pop_fused, "pop_two_op": workload_pop_two_op,
             "long": workload_long, "layer5": workload_layer5}


def time_steps(step, n):
    """n steps bracketed by synchronisations -> (wall ms per step, forward ms, backward ms from the events)."""
    import torch
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(n)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(n):
        step(events[i])
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / n
    return wall, sum(e[0].elapsed_time(e[1]) for e in events) / n, sum(e[1].elapsed_time(e[2]) for e in events) / n


def settle_and_time(step, args, n, warm):
    if args.spin_up > 0:   # (inputs are made on the host: the device idled meanwhile and its clocks fell back)
        spin_up(step, args.spin_up)
    for _ in range(warm):
        step()
    return time_steps(step, n)


def step_roofline(leg, info, ms, fwd_ms, bwd_ms, kernels):
    """The HBM roofline of a whole step of a workload: its algorithmic bytes (every tensor once per pass) over
    its time, the forward and backward parts from events on the launch stream, and the HBM traffic of all
    its launches as the counters gave it (read from profiles/)."""
    b_fwd, b_bwd = info["bytes"]
    traffic, commit = profiled_step_traffic(leg)
    gbs = lambda nbytes, t: round(nbytes / (t * 1e-3) / 1e9, 1)
    return {
        "bound": "hbm", "achieved": gbs(b_fwd + b_bwd, ms), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round((b_fwd + b_bwd) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "traffic": traffic, "traffic_measured_at_commit": commit,
        "algorithmic_bytes_per_step": b_fwd + b_bwd, "kernels": kernels,
        "forward_ms": round(fwd_ms, 4), "forward_achieved": gbs(b_fwd, fwd_ms),
        "backward_ms": round(bwd_ms, 4), "backward_achieved": gbs(b_bwd, bwd_ms),
    }


def gpu_leg(args):
    import torch
    from flash_pop_amd import _lib

    lib = _lib.load()   # fail loudly before any timing if the HIP library is missing
    dev = "cuda:0"
    step, info = workload_headline(dev)
    B, T, H, dk, dv = info["shape"]

    # the flags as given, from an idle device (the inputs were just made on the host): W warm-up steps, K timed
    for _ in range(args.warmup):
        step()
    cold_ms, cold_fwd, cold_bwd = time_steps(step, args.steps)
    # ... and with the device's clocks settled
    spin_steps = spin_up(step, args.spin_up) if args.spin_up > 0 else 0
    for _ in range(args.warmup):
        step()
    ms_per_step, fwd_ms, bwd_ms = time_steps(step, args.steps)

    f_fwd, f_bwd = info["flops"]
    b_fwd, b_bwd = info["bytes"]
    tflops = (f_fwd + f_bwd) / (ms_per_step * 1e-3) / 1e12
    # A step is two launches: the forward pass and the whole backward in one kernel, which is the
    # dominant one (about 70 % of the step).  Its roofline: the bytes the backward has to move
    # (q, k, v, dO in; dq, dk, dv out, each once) over its launch duration.
    bwd_kernel = "retention_bwd_fused_kernel<128, 128, 0>"
    bwd_gbs = b_bwd / (bwd_ms * 1e-3) / 1e9
    fwd_gbs = b_fwd / (fwd_ms * 1e-3) / 1e9
    step_gbs = (b_fwd + b_bwd) / (ms_per_step * 1e-3) / 1e9
    traffic, traffic_commit = profiled_traffic(bwd_kernel.split("<")[0])

    out = {
        "metric": "fwd+bwd retention TFLOP/s, B=8 H=16 T=4096 d=128 bf16",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "config 2: chunked retention fwd+bwd, B=8 H=16 T=4096 dk=dv=128 chunk 64, bf16 in / fp32 accumulate"},
        "tokens_per_s": round(B * T / (ms_per_step * 1e-3), 1),
        "fwd_ms": round(fwd_ms, 4),
        "bwd_ms": round(bwd_ms, 4),
        "mfma_frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
        # the same time priced with only the causal half of every C x C tile counted (C -> (C + 1) / 2)
        "tflops_causal_only": round(sum(algorithmic_flops(B, T, H, dk, dv, C=(CHUNK + 1) / 2)) / (ms_per_step * 1e-3) / 1e12, 2),
        # the same W + K steps started from an idle device, before the spin-up: what a cold call costs
        "ms_per_step_cold": round(cold_ms, 4),
        "value_cold": round((f_fwd + f_bwd) / (cold_ms * 1e-3) / 1e12, 2),
        "fwd_ms_cold": round(cold_fwd, 4),
        "bwd_ms_cold": round(cold_bwd, 4),
        "set_up": {"spin_up_seconds": args.spin_up, "spin_up_steps": spin_steps,
                   "why": "device clocks settle over the first ~50 steps from idle; `value` is timed after this much of "
                          "the same work and the --warmup steps, `value_cold` / `ms_per_step_cold` before it"},
        "library_version": lib.fp_version(),
        "roofline": {
            "bound": "hbm",
            "kernel": bwd_kernel + " (one launch = the whole backward of a step: dq, dk, dv)",
            "achieved": round(bwd_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(bwd_gbs / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_measured_at_commit": traffic_commit,
            # the counters' bytes over this run's launch time: the rate at which the kernel really streams
            "achieved_on_measured_traffic": round(traffic / (bwd_ms * 1e-3) / 1e9, 1) if traffic else None,
            "launch_ms": round(bwd_ms, 4),
            "algorithmic_bytes_per_launch": b_bwd,
            # the other launch of a step and the step as a whole, priced the same way
            "forward_kernel": "retention_pass_ws_kernel<128, 1, 1> (the forward pass, leaving its state every 512 tokens for the backward)",
            "forward_launch_ms": round(fwd_ms, 4),
            "forward_algorithmic_bytes_per_launch": b_fwd,
            "forward_achieved": round(fwd_gbs, 1),
            "forward_frac": round(fwd_gbs / HBM_PEAK_GBS, 4),
            "step_algorithmic_bytes": b_fwd + b_bwd,
            "step_achieved": round(step_gbs, 1),
            "step_frac": round(step_gbs / HBM_PEAK_GBS, 4),
        },
    }
    del step
    n_other, warm_other = max(12, args.steps // 4), max(5, args.warmup // 2)

    if not args.no_pop:
        ratio = lambda ms, i: round((ms / i["tokens"]) / (ms_per_step / i["tokens_context"]), 3)
        step, i = workload_pop_two_op(dev)
        two_ms, two_fwd, two_bwd = settle_and_time(step, args, n_other, warm_other)
        two = {
            "path": "flash_pop_retention, torch.cat of the block states, fused_chunk_retention (the reference's call sequence)",
            "ms_per_step": round(two_ms, 4),
            "cost_per_token_vs_plain": ratio(two_ms, i),
            "roofline": step_roofline("pop_two_op", i, two_ms, two_fwd, two_bwd,
                                      "context forward / backward with block states, suffix-batch forward / backward, torch's cat and slice copies"),
        }
        del step
        step, i = workload_pop_fused(dev)
        fused_ms, fused_fwd, fused_bwd = settle_and_time(step, args, n_other, warm_other)
        out["pop"] = {
            "workload": "config 4: POP context (64-token blocks) + 65 suffixes x 16 tokens per sequence, fwd+bwd",
            "tokens": i["tokens"],
            "ms_per_step": round(fused_ms, 4),
            "cost_per_token_vs_plain": ratio(fused_ms, i),
            "path": "flash_pop_retention_with_suffixes (suffixes read the state at their boundary in place: no block state in HBM)",
            "roofline": step_roofline("pop_fused", i, fused_ms, fused_fwd, fused_bwd,
                                      "suffix walk of the pass kernel (forward); fused backward with folded suffixes + suffix_intra_bwd_kernel"),
            "two_op_path": two,
        }
        del step
    if not args.no_long:
        step, i = workload_long(dev)
        long_ms, long_fwd, long_bwd = settle_and_time(step, args, n_other, warm_other)
        B3, T3, H3, dk3, dv3 = i["shape"]
        out["long_context"] = {
            "workload": "config 3: B=2 H=8 T=16384 dk=128 dv=256, carried state, fwd+bwd incl. dS0",
            "ms_per_step": round(long_ms, 4),
            "tflops": round(sum(i["flops"]) / (long_ms * 1e-3) / 1e12, 2),
            "algorithmic_gbs": round(sum(i["bytes"]) / (long_ms * 1e-3) / 1e9, 1),
            "segments_per_sequence": lib.fp_retention_workspace_bytes(B3, T3, H3, dk3, dv3) // (4 * B3 * H3 * dk3 * dv3),
            "roofline": step_roofline("long", i, long_ms, long_fwd, long_bwd,
                                      "split-sequence entry points: state-only passes, segment scans, forward pass and the gradient kernels on the segments"),
        }
        del step
    if not args.no_layer5:
        step, i = workload_layer5(dev)
        l5_ms, l5_fwd, l5_bwd = settle_and_time(step, args, n_other, warm_other)
        out["model_layer"] = {
            "workload": "the retention op of one layer of config 5: fused POP step, B=8 T=2048 H=12 dk=64 dv=128, "
                        "64-token blocks, 33 suffixes x 16 tokens per sequence, fwd+bwd",
            "tokens": i["tokens"],
            "ms_per_step": round(l5_ms, 4),
            "roofline": step_roofline("layer5", i, l5_ms, l5_fwd, l5_bwd,
                                      "suffix walk of the pass kernel (forward); the backward kernels of this shape"),
        }
        del step
    if not args.no_layer:
        out["layer_ops"] = layer_leg(args, dev)
    if not args.no_model:
        out["model"] = model_leg(args, dev)
    return out


def layer_leg(args, dev):
    """The two elementwise stages around the op at config 2's tensor shapes (B=8 T=4096 H=16 d=128):
    time per launch and algorithmic bytes per second (every tensor once), next to the same
    stage as eager torch (the reference's call sequence)."""
    import torch
    import torch.nn.functional as F
    if TESTS not in sys.path:
        sys.path.insert(0, TESTS)
    import model_harness as mh
    from flash_pop_amd import XPos, gated_group_norm

    B, T, H, d = 8, 4096, 16, 128
    g = torch.Generator(device=dev).manual_seed(7)
    q, k, r, gate, d_out = (torch.randn(B, T, H, d, generator=g, device=dev).to(torch.bfloat16) for _ in range(5))
    gate, d_out = gate.flatten(-2), d_out.flatten(-2)
    tensor_bytes = q.numel() * 2
    xpos = XPos(d)

    def timed(fn, n=max(5, args.steps // 2)):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    def torch_norm_gate():
        n = F.group_norm(r.reshape(B * T, H * d).float(), H, eps=1e-6).to(torch.bfloat16).reshape(B, T, H * d)
        return n * F.silu(gate)

    rl, gl = r.clone().requires_grad_(), gate.clone().requires_grad_()
    out = gated_group_norm(rl, gl, 1e-6)
    rows = []
    for name, fn, eager, tensors in (
            ("rotary_qk_kernel", lambda: xpos(q, k, 0), lambda: (mh.rotate(q, 0), mh.rotate(k, 0)), 4),
            ("gated_norm_fwd_kernel", lambda: gated_group_norm(r, gate, 1e-6), torch_norm_gate, 3),
            ("gated_norm_bwd_kernel", lambda: torch.autograd.grad(out, [rl, gl], d_out, retain_graph=True), None, 5)):
        ms = timed(fn)
        row = {"kernel": name, "ms": round(ms, 4), "algorithmic_gbs": round(tensors * tensor_bytes / (ms * 1e-3) / 1e9, 1),
               "hbm_frac": round(tensors * tensor_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 3)}
        if eager is not None:
            row["eager_torch_ms"] = round(timed(eager, n=5), 4)
        rows.append(row)
    return {"workload": "B=8 T=4096 H=16 d=128 bf16: q, k rotated in one launch; per-head norm + swish gate, fwd and bwd",
            "kernels": rows}


def model_leg(args, dev):
    """Config 5: a random-init 12-layer POP-RetNet decoder (tests/model_harness.py) on the HIP ops:
    one POP training step (fwd+bwd, B=8, T=2048 in 64-token blocks with 16-token suffixes), then
    256 recurrent decode steps from the states it leaves."""
    import torch
    if TESTS not in sys.path:
        sys.path.insert(0, TESTS)
    import model_harness as mh

    cfg = mh.HarnessConfig()
    B, T, decode_steps = 8, 2048, 256
    backend = mh.HipBackend()
    model = mh.build(cfg, seed=0, device=dev)
    batch = mh.synthetic_batch(cfg, B, T, seed=1, device=dev)

    def train_step():
        model.zero_grad(set_to_none=True)
        loss, _, _, states = mh.pop_loss(model, backend, batch)
        loss.backward()
        return states

    def time_train():
        for _ in range(2):
            train_step()
        torch.cuda.synchronize()
        n = max(3, args.steps // 10)
        t0 = time.perf_counter()
        for _ in range(n):
            states = train_step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / n, states

    backend = mh.HipBackend(layer_ops=False)     # rotary embedding and norm + gate as eager torch
    eager_ms, _ = time_train()
    backend = mh.HipBackend()
    train_ms, states = time_train()

    states = [s.detach() for s in states]
    token = batch[0][:, -1]
    with torch.no_grad():
        for i in range(8):
            logits, states = model.recurrent(backend, token, states, T + i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(decode_steps):
            logits, states = model.recurrent(backend, token, states, T + 8 + i)
            token = logits.argmax(-1)
        torch.cuda.synchronize()
    decode_ms = (time.perf_counter() - t0) * 1e3 / decode_steps

    # the same step captured once in a HIP graph and replayed
    dec = mh.GraphedGreedyDecoder(model, backend, states, token, T + 8 + decode_steps)
    for _ in range(8):
        dec.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(decode_steps):
        dec.step()
    torch.cuda.synchronize()
    graph_ms = (time.perf_counter() - t0) * 1e3 / decode_steps
    tokens = B * T + B * (T // cfg.block + 1) * cfg.sfx_len
    return {
        "workload": "config 5: 12-layer POP-RetNet decoder d_model=768 H=12 dk=64 dv=128 FFN=3072 vocab=32000, "
                    "bf16, B=8 T=2048, 64-token blocks, 16-token suffixes; eager torch around the HIP ops "
                    "(retention, rotary embedding of q and k, per-head norm + gate)",
        "train_step_ms": round(train_ms, 2),
        "train_step_ms_retention_ops_only": round(eager_ms, 2),
        "train_tokens_per_s": round(tokens / (train_ms * 1e-3), 1),
        "decode_steps": decode_steps,
        "decode_ms_per_step": round(graph_ms, 3),
        "decode_tokens_per_s": round(B / (graph_ms * 1e-3), 1),
        "decode_path": "one decode step captured in a HIP graph (12 layers, decode-step kernel in place), replayed",
        "decode_eager_ms_per_step": round(decode_ms, 3),
    }


def cpu_leg(sample_batch=8, reps=3):
    """The oracle (chunk 64, fp32, torch autograd for the backward) on the host cores, on
    `sample_batch` of the 8 sequences of config 2.  Threads: what torch takes from the
    environment (OMP_NUM_THREADS, else every core the process may run on)."""
    import torch
    if TESTS not in sys.path:
        sys.path.insert(0, TESTS)
    import oracle
    import helpers as hp

    allowed = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    if "OMP_NUM_THREADS" not in os.environ:
        torch.set_num_threads(allowed)
    B, T, H, dk, dv = sample_batch, 4096, 16, 128, 128
    decays = head_decays(H)
    assert decays == oracle.head_decays(H)
    q, k, v, s = make_inputs(B, T, H, dk, dv, seed=0, state_std=0.0)
    d_o, = make_cotangents([(B, T, H, dv)], seed=1)
    times = []
    for i in range(reps + 1):
        t0 = time.perf_counter()
        hp.oracle_plain(q, k, v, s, decays, d_o, None, chunk=CHUNK)
        if i:
            times.append(time.perf_counter() - t0)
    sec = sorted(times)[len(times) // 2]
    f_fwd, f_bwd = algorithmic_flops(B, T, H, dk, dv)
    return {
        "value": round((f_fwd + f_bwd) / sec / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "host_cores": os.cpu_count(),
        "cores_allowed": allowed,
        "omp_num_threads_env": os.environ.get("OMP_NUM_THREADS"),
        "kind": "port",
        "sample": f"{B} of the 8 sequences of config 2 (H=16 T=4096 d=128), fp32, chunk 64, fwd+bwd, "
                  f"median of {reps} after 1 warm-up, {sec:.2f} s each",
        "tokens_per_s": round(B * T / sec, 1),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--spin-up", type=float, default=SPIN_UP_SECONDS,
                    help="seconds of the benchmarked step run during set-up so that the device clocks have settled (0: none)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-pop", action="store_true", help="skip the POP (config 4) timing")
    ap.add_argument("--no-long", action="store_true", help="skip the long-context (config 3) timing")
    ap.add_argument("--no-layer5", action="store_true", help="skip the timing of config 5's retention op on its own")
    ap.add_argument("--no-layer", action="store_true", help="skip the timing of the rotary / norm + gate kernels")
    ap.add_argument("--profile-leg", choices=sorted(WORKLOADS), default=None,
                    help="run exactly --steps steps of one workload and nothing else (for the rocprofv3 runs)")
    ap.add_argument("--no-model", action="store_true", help="skip the model-level (config 5) timing")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 1 GiB device copy (scales the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.copy_calibration:
        import torch
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": src.numel()}))
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")
    if args.profile_leg:
        import torch
        step, _ = WORKLOADS[args.profile_leg]("cuda:0")
        if args.spin_up > 0:   # for kernel traces at settled clocks; counter runs pass --spin-up 0
            spin_up(step, args.spin_up)
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        print(json.dumps({"profile_leg": args.profile_leg, "steps": args.steps}))
        return
    out = gpu_leg(args)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_leg()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()

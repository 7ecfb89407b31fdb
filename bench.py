"""Benchmark of the two hot paths on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle N] [--path both|attn|lion|next|copy|clock|power|ablations]
                    [--no-cpu-baseline] [--headline-only]

Prints ONE JSON line. The headline value is the attention forward throughput at B=2 H=16 S=8192 D=128 bf16 causal
(FLOPs counted as 2*B*H*S^2*D); the fused Lion step over 1,308,622,848 fp32 parameters with bf16 momentum (16 bytes
per parameter) is reported in the "lion" object of the same line, each with its roofline and a CPU baseline timed on
this host's cores. Beside them, not part of the headline: the attention backward of the same shape ("attn_bwd"), the
other three benchmark configurations ("configs": GPT-2-small attention forward, GPT-2-small Lion, fp16 non-causal
attention forward at B=16 H=32 S=2048 D=128), and the rate of the vendor library's plain bf16 GEMM on random operands
on the same box ("library_gemm": what MFMA code reaches here at all), and three variations of the headline launch
("headline_variants": the same shape non-causal, the same causal launch on all-zero operands, and head_dim 64 at
B=2 H=32 S=8192 causal) with the ratio of the causal time to half the non-causal time, and the headline launch and the
B=16 H=32 S=2048 launch once more with one work item per workgroup (attn.keep_on 0) instead of workgroups that walk
their share of the items.

`--path next` times what lies around the two headline kernels with the same machinery: attention forward, backward and
forward+backward on the reference's own benchmark matrix (1 x 12 heads x {2048, 4096, 8192} x 128, bf16, with and
without causal mask, dropout 0.1 and a [B,1,1,S] bias; the reference's published A100 timings are quoted beside them),
and the fused Lion step at the reference's benchmark sizes (8192 and 8192^2 elements, all-fp16 and all-bf16) and at
1.3 B parameters for all-bf16 and fp32-momentum tensors.

Every timed section is preceded by a clock-settle phase of --settle launches of the same step (default 100, reported
under "settle"), which is not part of the W warm-up steps: after idling, the GPU's clocks take a few dozen launches
to settle (the per-launch time of the attention kernel wanders by 25 % over the first 30 launches, then stays within
1 %), so without it the result would depend on the caller's --warmup.

All inputs are drawn from a CPU torch.Generator in fp32 with the seeds the configurations name, cast, and copied to the
GPU before timing starts; nothing crosses PCIe in a timed region.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_MFMA_TFLOPS = 2500.0     # MI355X dense bf16/fp16
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E
TRAFFIC_SOURCE = ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this workload, recorded in "
                  "profiles/hbm_traffic_pmc_attn_S8192_lion_1p3B.txt; a constant read from profiles/hbm_traffic.json, not measured by this run")


def _measured_traffic(key):
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this workload (the runs and the
    scaling against a plain copy are in profiles/hbm_traffic_pmc_*.txt); None when that file is absent."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            return json.load(f).get(key)
    except OSError:
        return None


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _host_threads():
    """Threads for the CPU baselines: the cores this process may run on, at most what OMP_NUM_THREADS allows."""
    n = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    try:
        n = min(n, int(os.environ["OMP_NUM_THREADS"]))
    except (KeyError, ValueError):
        pass
    return max(1, n)


def _events(n):
    import torch

    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _settle(step, launches, steady=0.015, min_seconds=1.0, max_seconds=4.0):
    """Untimed-for-the-result launches of `step` so that the clocks are where a sustained run has them: blocks of
    `launches`, repeated until the phase has lasted `min_seconds` and the median launch time of a block is within `steady`
    of the block before it (`max_seconds` at most). On some boxes of the pool the chip runs its first 0.2 s under
    load fast, the next half second 15 % slower and settles in between after a second or two; a section that is timed
    0.1 s after the load began measures that transient, not the run. The first and last per-launch times and the block
    medians are reported to show what the phase did."""
    import torch

    if launches <= 0:
        return {"launches": 0}
    medians, first, ms_max = [], None, 0.0
    t_begin = time.perf_counter()
    while True:
        ev = _events(launches + 1)
        ev[0].record()
        for i in range(launches):
            step()
            ev[i + 1].record()
        torch.cuda.synchronize()
        ms = [ev[i].elapsed_time(ev[i + 1]) for i in range(launches)]
        k = max(1, min(5, launches // 2))
        if first is None:
            first = sum(ms[:k]) / k
        ms_max = max(ms_max, max(ms))
        medians.append(sorted(ms)[launches // 2])
        elapsed = time.perf_counter() - t_begin
        if elapsed >= max_seconds or (elapsed >= min_seconds and len(medians) >= 2 and abs(medians[-1] - medians[-2]) <= steady * medians[-2]):
            break
    shown = medians if len(medians) <= 12 else medians[:6] + medians[-6:]
    return {"launches": launches * len(medians), "seconds": round(time.perf_counter() - t_begin, 3), "ms_first": first,
            "ms_last": sum(ms[-k:]) / k, "ms_max": ms_max, "block_medians_ms": [round(m, 5) for m in shown]}


def _time_steps(step, steps, warmup, settle=0, before_each=None, wall_without_events=False):
    """`settle` clock-settle launches, W untimed steps, then K timed steps bracketed by synchronize; per-launch durations
    from HIP events recorded on the stream the kernels are launched on (torch's current stream). `before_each(i)`, if
    given, runs before timed step i outside its pair of events (fresh inputs for the step; only then are the events
    pairs). With `wall_without_events` the wall time per step comes from K further steps with no events between them
    (for kernels of a few tens of microseconds, where the event records are a sizeable part of a step)."""
    import gc

    import torch

    # Python's cycle collector stays out of the timed steps: a full collection in this process takes tens of
    # milliseconds of host time, which the events around a 30-microsecond launch see as the GPU waiting. It runs before
    # the settle phase, and the events are made there too, so that between the last warm-up step and the first timed one
    # the chip is idle for no longer than the synchronize the contract asks for: on some boxes of the pool every pause
    # under load is followed by some twenty launches that take up to 35 % longer.
    gc.collect()
    gc_was_on = gc.isenabled()
    gc.disable()
    marks = _events(steps + 1)
    starts, ends = (_events(steps), _events(steps)) if before_each is not None else (None, None)
    try:
        info = _settle(step, settle)
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        wall_plain = None
        if wall_without_events:
            t0 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            wall_plain = (time.perf_counter() - t0) * 1e3 / steps
        if before_each is None:
            # one event after every step (and one in front of the first): a launch's time runs from the end of the launch
            # before it to its own end
            t0 = time.perf_counter()
            marks[0].record()
            for i in range(steps):
                step()
                marks[i + 1].record()
            torch.cuda.synchronize()
            wall_ms = (time.perf_counter() - t0) * 1e3
            per_launch = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]
        else:
            t0 = time.perf_counter()
            for i in range(steps):
                before_each(i)
                starts[i].record()
                step()
                ends[i].record()
            torch.cuda.synchronize()
            wall_ms = (time.perf_counter() - t0) * 1e3
            per_launch = [starts[i].elapsed_time(ends[i]) for i in range(steps)]
    finally:
        if gc_was_on:
            gc.enable()
    info = dict(info, kernel_ms_median=sorted(per_launch)[steps // 2])
    if steps <= 64:
        info["timed_launches_ms"] = [round(x, 4) for x in per_launch]   # (beside the settle blocks: shows a chip still changing clocks)
    return (wall_plain if wall_plain is not None else wall_ms / steps), sum(per_launch) / steps, min(per_launch), info


def _attn_inputs(B, H, S, D, dtype, dev, seed=0):
    import torch

    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(B, H, S, D, generator=g).to(dtype).to(dev) for _ in range(3)), g


KERNEL_NAMES = {0: "rows128", 1: "rows128_exact", 8: "rows128_pipelined", 16: "rows256_w8", 32: "rows256_w4"}


def _attn_rate(B, H, S, D, dtype, causal, steps, warmup, settle, operands="normal", backward=False):
    """One attention-forward configuration through multi_head_attention: a dict with the wall time per step (steps with
    no events between them), the kernel time (events), the rate by both and which kernel ran; with `backward`, the same
    for the backward (dQ + dK/dV launches, five-GEMM FLOP count) under "bwd". `operands`: "normal" (standard normal from
    the CPU generator, seed 0) or "zero"."""
    import ctypes

    import torch

    from fast_ops.flash_attention.flash_attention import multi_head_attention
    from fast_ops_amd import _lib
    from fast_ops_amd.flash_attention.flash_attention import attn_bwd_strided

    (q, k, v), g = _attn_inputs(B, H, S, D, dtype, "cuda:0")
    if operands == "zero":
        q, k, v = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    scale = 1.0 / (D ** 0.5)
    flops = (2.0 if causal else 4.0) * B * H * S * S * D
    out = {}

    def fwd():
        out["o"], out["lse"] = multi_head_attention(q, k, v, causal=causal, softmax_scale=scale, return_lse=True)

    ms_step, ms_kernel, ms_min, info = _time_steps(fwd, steps, warmup, settle, wall_without_events=True)
    I3 = ctypes.c_int64 * 3
    kernel = _lib.load().fo_attn_fwd_kernel(B, H, S, S, D, I3(*k.stride()[:3]), I3(*v.stride()[:3]), int(causal), 0, 0)
    res = {
        "workload": f"attention fwd B={B} H={H} S={S} D={D} {'bf16' if dtype == torch.bfloat16 else 'fp16'} {'causal' if causal else 'non-causal'}"
                    + (", all-zero operands" if operands == "zero" else ""),
        "ms_per_step": ms_step, "kernel_ms_avg": ms_kernel, "kernel_ms_min": ms_min, "value": flops / (ms_step * 1e-3) / 1e12, "unit": "TFLOP/s",
        "achieved": flops / (ms_kernel * 1e-3) / 1e12, "frac": flops / (ms_kernel * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "flops_per_launch": flops,
        "kernel": KERNEL_NAMES.get(kernel, str(kernel)), "kernel_ms_median": info["kernel_ms_median"],
        "frac_median": flops / (info["kernel_ms_median"] * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "settle": info,
    }
    if backward:
        go = torch.randn(B, H, S, D, generator=g).to(dtype).to("cuda:0")
        o_fix, lse_fix = out["o"], out["lse"]
        bflops = 2.5 * flops
        b_step, b_kernel, b_min, b_info = _time_steps(lambda: attn_bwd_strided(q, k, v, o_fix, lse_fix, go, (0, 1, 2, 3), causal, scale),
                                                      steps, warmup, settle // 2, wall_without_events=True)
        res["bwd"] = {"ms_per_step": b_step, "kernel_ms_avg": b_kernel, "kernel_ms_min": b_min, "kernel_ms_median": b_info["kernel_ms_median"], "value": bflops / (b_step * 1e-3) / 1e12, "unit": "TFLOP/s",
                      "frac": bflops / (b_kernel * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS,
                      "frac_median": bflops / (b_info["kernel_ms_median"] * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "flops_per_launch": bflops,
                      "what": "dQ + dK/dV launches of the same shape, FLOPs by the five-GEMM count"}
    return res


def bench_attention(steps, warmup, settle, cpu_baseline, extras):
    import torch

    from fast_ops.flash_attention.flash_attention import multi_head_attention

    B, H, S, D = 2, 16, 8192, 128
    dev = "cuda:0"
    (q, k, v), g = _attn_inputs(B, H, S, D, torch.bfloat16, dev)
    scale = 1.0 / (D ** 0.5)
    flops = 2.0 * B * H * S * S * D      # causal-halved 4*B*H*S^2*D
    out = {}

    def step():
        out["o"], out["lse"] = multi_head_attention(q, k, v, causal=True, softmax_scale=scale, return_lse=True)

    ms_step, ms_kernel, ms_min, info = _time_steps(step, steps, warmup, settle)
    res = {
        "value": flops / (ms_step * 1e-3) / 1e12,
        "ms_per_step": ms_step,
        "settle": info,
        "roofline": {
            "bound": "mfma", "achieved": flops / (ms_kernel * 1e-3) / 1e12, "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s",
            "frac": flops / (ms_kernel * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "traffic": _measured_traffic("attn"), "traffic_source": TRAFFIC_SOURCE,
            "kernel_ms_avg": ms_kernel, "kernel_ms_min": ms_min, "flops_per_launch": flops,
        },
        "workload": f"attention fwd B={B} H={H} S={S} D={D} bf16 causal, scale 1/sqrt({D})",
    }
    if extras:
        # the backward of the same workload (dQ, dK, dV; two launches), reported beside the headline, not part of it
        from fast_ops_amd.flash_attention.flash_attention import attn_bwd_strided

        go = torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(dev)
        o_fix, lse_fix = out["o"], out["lse"]
        bwd_flops = 5.0 * B * H * S * S * D      # causal-halved 10*B*H*S^2*D (five GEMMs; the kernels recompute two more)
        b_step, b_kernel, b_min, b_info = _time_steps(lambda: attn_bwd_strided(q, k, v, o_fix, lse_fix, go, (0, 1, 2, 3), True, scale), steps, warmup, settle // 2)
        res["bwd"] = {
            "value": bwd_flops / (b_step * 1e-3) / 1e12, "unit": "TFLOP/s", "ms_per_step": b_step, "settle": b_info,
            "roofline": {"bound": "mfma", "achieved": bwd_flops / (b_kernel * 1e-3) / 1e12, "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s",
                         "frac": bwd_flops / (b_kernel * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "traffic": None,
                         "kernel_ms_avg": b_kernel, "kernel_ms_min": b_min, "flops_per_launch": bwd_flops},
            "workload": "attention bwd (dQ + dK/dV kernels) of the same shape, FLOPs by the five-GEMM count",
        }
        del go, o_fix, lse_fix
        # yardstick, not part of the headline: the vendor library's plain bf16 GEMM on the same box with the same kind of
        # data. Under a full-chip MFMA load the clock follows the power drawn, which depends on the operand bits (all-zero
        # operands run a third faster than random ones), so the published peak is not what random data can reach.
        n = 8192
        ga, gb = (torch.randn(n, n, generator=g).to(torch.bfloat16).to(dev) for _ in range(2))
        _, g_kernel, _, _ = _time_steps(lambda: torch.matmul(ga, gb), 20, 20, settle // 2)
        res["library_gemm"] = {
            "value": 2.0 * n ** 3 / (g_kernel * 1e-3) / 1e12, "unit": "TFLOP/s", "frac_of_peak": 2.0 * n ** 3 / (g_kernel * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS,
            "what": f"torch.matmul (hipBLASLt) bf16 {n}x{n}x{n}, standard normal operands, same box, timed after the attention runs",
        }
        del ga, gb
    if cpu_baseline:
        # bounded sample: all (batch, head) slices of the same workload through the oracle's fp32 vanilla path on all host
        # cores, stopped after about 15 s; the rate is that of the slices that were finished
        from oracle.attention_oracle import attention_fwd_oracle

        torch.set_num_threads(_host_threads())
        qc, kc, vc = (t.cpu() for t in (q, k, v))
        attention_fwd_oracle(qc[:1, :1, :1024], kc[:1, :1, :1024], vc[:1, :1, :1024], causal=True, softmax_scale=scale)   # warm-up
        n_sl, t0 = 0, time.perf_counter()
        for bb in range(B):
            for hh in range(H):
                if time.perf_counter() - t0 > 15.0:
                    break
                attention_fwd_oracle(qc[bb:bb + 1, hh:hh + 1], kc[bb:bb + 1, hh:hh + 1], vc[bb:bb + 1, hh:hh + 1], causal=True, softmax_scale=scale)
                n_sl += 1
        dt = time.perf_counter() - t0
        res["cpu_baseline"] = {
            "value": n_sl * 2.0 * S * S * D / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "cpu_model": _cpu_model(), "kind": "port",
            "sample": f"{n_sl} of {B * H} (batch, head) slices of the same shape, fp32 vanilla softmax(QK^T)V on the host, {dt:.2f} s",
        }
    del q, k, v
    out.clear()
    torch.cuda.empty_cache()
    if extras:
        # the headline launch varied one thing at a time, on the same box right after it: what the causal mask costs
        # against half a non-causal launch, what the operand bits cost (all-zero operands toggle nothing in the
        # multipliers: the same instruction stream at the clock the power limit then allows), and head_dim 64
        hv = {
            "causal": _attn_rate(B, H, S, D, torch.bfloat16, True, steps, warmup, settle),
            "noncausal": _attn_rate(B, H, S, D, torch.bfloat16, False, steps, warmup, settle),
            "zero_operands": _attn_rate(B, H, S, D, torch.bfloat16, True, steps, warmup, settle, operands="zero"),
            "zero_operands_noncausal": _attn_rate(B, H, S, D, torch.bfloat16, False, steps, warmup, settle, operands="zero"),
            "head_dim_64": _attn_rate(2, 32, 8192, 64, torch.bfloat16, True, steps, warmup, settle),
        }
        hv["causal_over_half_noncausal"] = hv["causal"]["kernel_ms_avg"] / (0.5 * hv["noncausal"]["kernel_ms_avg"])
        # what the workgroups' walk over the work items is worth (attn.keep_on 0: one item per workgroup, no copies ahead
        # for the next query block), at the headline shape and at B=16 H=32 S=2048 fp16 non-causal, whose query blocks are short
        from fast_ops_amd import _lib

        _lib.tune_set("attn.keep_on", 0)
        try:
            hv["causal_one_item_per_workgroup"] = _attn_rate(B, H, S, D, torch.bfloat16, True, steps, warmup, settle)
            hv["config_5a_one_item_per_workgroup"] = _attn_rate(16, 32, 2048, 128, torch.float16, False, steps, warmup, settle)
        finally:
            _lib.tune_set("attn.keep_on", -1)
        res["headline_variants"] = hv
        torch.cuda.empty_cache()
        # the other attention configurations: report only
        res["configs"] = {
            "2_attn_fwd_gpt2_small": _attn_rate(8, 12, 1024, 64, torch.bfloat16, True, steps, warmup, settle, backward=True),
            "5a_attn_fwd_throughput": _attn_rate(16, 32, 2048, 128, torch.float16, False, steps, warmup, settle, backward=True),
        }
        torch.cuda.empty_cache()
    return res


GPT2_SMALL_SHAPES = ([(50257, 768), (1024, 768)]
                     + [s for _ in range(12) for s in [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,), (768,), (768,), (768, 3072), (3072,), (3072, 768), (768,)]]
                     + [(768,), (768,)])
LION_LARGE_SHAPES = [(2048, 8192)] * 39 + [(8192, 2048)] * 39
LION_HP = dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)


def _lion_setup(shapes, dev):
    """Parameters ~ N(0, 0.02) and bf16 momentum ~ N(0, 1e-3) from a CPU generator seeded 0 (parameters first, then
    momenta), gradients ~ N(0, 1e-2) from seed 1000 (the first step's); copied to the GPU."""
    import torch

    from fast_ops.lion.lion_optimizer import Lion

    gen = torch.Generator().manual_seed(0)
    params = [torch.nn.Parameter((torch.randn(s, generator=gen) * 0.02).to(dev)) for s in shapes]
    opt = Lion(params, **LION_HP)
    for p in params:
        opt.state[p]["exp_avg"] = (torch.randn(p.shape, generator=gen) * 1e-3).to(torch.bfloat16).to(dev)
    ggen = torch.Generator().manual_seed(1000)
    for p in params:
        p.grad = (torch.randn(p.shape, generator=ggen) * 1e-2).to(dev)
    return params, opt


def bench_lion(steps, warmup, settle, cpu_baseline, extras):
    import torch

    dev = "cuda:0"
    res_small = None
    if extras:
        # configuration 3: the GPT-2-small parameter set, 10 steps with fresh seeded gradients each step (copied into the
        # gradient tensors between the timed steps, outside their events)
        params, opt = _lion_setup(GPT2_SMALL_SHAPES, dev)
        n_small = sum(p.numel() for p in params)
        assert len(params) == 148 and n_small == 124439808
        fresh = []
        for s in range(10):
            gg = torch.Generator().manual_seed(1000 + s)
            fresh.append((torch.randn(n_small, generator=gg) * 1e-2).to(dev))

        views = []
        for s_ in range(10):
            at, vs = 0, []
            for p in params:
                vs.append(fresh[s_][at:at + p.numel()].view(p.shape))
                at += p.numel()
            views.append(vs)
        grads = [p.grad for p in params]

        def new_grads(i):
            torch._foreach_copy_(grads, views[i])

        s_step, s_kernel, s_min, s_info = _time_steps(opt.step, 10, warmup, settle, before_each=new_grads)
        res_small = {
            "workload": f"fused Lion step, GPT-2-small set: {len(params)} tensors = {n_small} fp32 params, bf16 momentum, 10 steps with fresh gradients",
            "ms_per_step": s_step, "kernel_ms_avg": s_kernel, "kernel_ms_min": s_min, "value": 16.0 * n_small / (s_kernel * 1e-3) / 1e9, "unit": "GB/s",
            "frac": 16.0 * n_small / (s_kernel * 1e-3) / 1e9 / PEAK_HBM_GBS, "bytes_per_launch": 16.0 * n_small, "settle": s_info,
            "steady_state": {"kernel_ms": s_info["ms_last"], "value": 16.0 * n_small / (s_info["ms_last"] * 1e-3) / 1e9, "unit": "GB/s",
                             "frac": 16.0 * n_small / (s_info["ms_last"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
                             "what": "back-to-back steps on unchanged gradients (the last launches of the settle phase)"},
            "note": "ms_per_step includes copying the fresh gradients; value and frac are from the events around each of the 10 steps "
                    "alone, which the GPU reaches before the host has issued the step, so they contain the host's time to issue it",
        }
        del opt, fresh, views, grads
        # the same parameter set in torch's default training loop: backward (autograd makes new gradient tensors), step(),
        # zero_grad() (set_to_none=True frees them). Host time of step() by the host's clock, kernel time by events around
        # the step, how often the chunk table had to be rebuilt, and what stays allocated after zero_grad().
        for p in params:
            p.grad = None
        from fast_ops.lion.lion_optimizer import Lion

        opt = Lion(params, **LION_HP)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        other0 = torch.cuda.memory_allocated() - sum(p.numel() * 4 for p in params)    # whatever else this process holds
        w = (torch.randn(n_small, generator=torch.Generator().manual_seed(7)) * 1e-2).to(dev)
        wv, at = [], 0
        for p in params:
            wv.append(w[at:at + p.numel()].view(p.shape))
            at += p.numel()
        host_us, kern_ms, held = [], [], []
        n_loop, skip = 30, 10
        ev = _events(2 * n_loop)
        rebuilds0 = None
        for it in range(n_loop):
            loss = sum([(p * v_).sum() for p, v_ in zip(params, wv)])
            loss.backward()
            del loss
            torch.cuda.synchronize()
            if it == skip:
                rebuilds0 = opt.table_rebuilds
            ev[2 * it].record()
            t0 = time.perf_counter()
            opt.step()
            host_us.append((time.perf_counter() - t0) * 1e6)
            ev[2 * it + 1].record()
            opt.zero_grad()
            torch.cuda.synchronize()
            kern_ms.append(ev[2 * it].elapsed_time(ev[2 * it + 1]))
            held.append(torch.cuda.memory_allocated() - other0 - n_small * (4 + 2 + 4))   # parameters, bf16 momenta, w
        hs, ks = sorted(host_us[skip:]), sorted(kern_ms[skip:])
        res_small["training_loop"] = {
            "what": "backward (autograd), step(), zero_grad() with set_to_none=True; figures over the last 20 of 30 iterations",
            "host_us_step_median": hs[len(hs) // 2], "host_us_step_min": hs[0], "step_ms_by_events_median": ks[len(ks) // 2],
            "table_rebuilds": opt.table_rebuilds - rebuilds0, "table_rebuilds_first_iterations": rebuilds0,
            "bytes_allocated_after_zero_grad_beyond_params_momenta_inputs": max(held[skip:]), "bytes_of_one_gradient_set": 4 * n_small,
        }
        del opt, params, w, wv
        torch.cuda.empty_cache()
    shapes = LION_LARGE_SHAPES
    n_params = sum(a * b for a, b in shapes)
    params, opt = _lion_setup(shapes, dev)
    nbytes = 16.0 * n_params
    ms_step, ms_kernel, ms_min, info = _time_steps(opt.step, steps, warmup, min(settle, 20))
    res = {
        "value": nbytes / (ms_step * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": ms_step, "dtype": "f32 params/grads, bf16 momentum", "settle": info,
        "roofline": {
            "bound": "hbm", "achieved": nbytes / (ms_kernel * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": nbytes / (ms_kernel * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": _measured_traffic("lion"), "traffic_source": TRAFFIC_SOURCE,
            "kernel_ms_avg": ms_kernel, "kernel_ms_min": ms_min, "bytes_per_launch": nbytes,
        },
        "workload": f"fused Lion step, {len(shapes)} tensors (39 x 2048x8192 + 39 x 8192x2048) = {n_params} fp32 params, bf16 momentum",
    }
    if res_small is not None:
        res["configs"] = {"3_lion_gpt2_small": res_small}
    if cpu_baseline:
        # bounded sample: 8 of the 78 tensors (134,217,728 parameters) through the four reference statements on all host
        # cores, 3 steps
        from oracle.lion_oracle import lion_step_torch

        torch.set_num_threads(_host_threads())
        n_t = 8
        ps = [params[i].detach().cpu().clone() for i in range(n_t)]
        gs = [params[i].grad.cpu().clone() for i in range(n_t)]
        ms = [opt.state[params[i]]["exp_avg"].cpu().clone() for i in range(n_t)]
        lion_step_torch(ps, gs, ms, LION_HP["lr"], LION_HP["betas"], LION_HP["weight_decay"])     # warm-up
        reps = 3
        t0 = time.perf_counter()
        for _ in range(reps):
            lion_step_torch(ps, gs, ms, LION_HP["lr"], LION_HP["betas"], LION_HP["weight_decay"])
        dt = (time.perf_counter() - t0) / reps
        n_el = sum(p.numel() for p in ps)
        res["cpu_baseline"] = {
            "value": 16.0 * n_el / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "cpu_model": _cpu_model(), "kind": "port",
            "sample": f"{n_t} of 78 tensors ({n_el} parameters), vanilla 4-statement PyTorch Lion step on the host, {dt * 1e3:.1f} ms per step, {reps} steps",
        }
    del opt, params
    torch.cuda.empty_cache()
    return res


# The reference's published timings on an A100 (fast_ops/flash_attention/README.md:76-175, column "Triton": its working
# implementation; fast_ops/lion/README.md:29-35, column "ours"), in microseconds, quoted beside this build's figures as
# context - other hardware, not a baseline of this benchmark. Keys: (seq_len, dropout_p, bias, causal) -> (fwd, bwd, fwd+bwd).
REF_A100_TRITON_US = {
    (2048, 0.0, 0, 0): (258.2, 1020.9, 1354.6), (2048, 0.0, 0, 1): (188.7, 730.1, 938.6), (2048, 0.1, 0, 0): (283.4, 826.7, 1132.7),
    (2048, 0.1, 0, 1): (230.7, 832.7, 1025.9), (2048, 0.0, 1, 0): (232.7, 870.6, 1129.0), (2048, 0.0, 1, 1): (192.1, 989.8, 1258.1),
    (2048, 0.1, 1, 0): (286.4, 857.1, 1161.1), (2048, 0.1, 1, 1): (233.0, 875.8, 1191.0),
    (4096, 0.0, 0, 0): (926.5, 2931.5, 3886.3), (4096, 0.0, 0, 1): (548.9, 2035.1, 2609.7), (4096, 0.1, 0, 0): (1102.2, 2965.1, 4084.2),
    (4096, 0.1, 0, 1): (674.3, 1847.9, 2539.7), (4096, 0.0, 1, 0): (901.7, 3130.8, 4055.6), (4096, 0.0, 1, 1): (565.9, 2453.2, 3036.3),
    (4096, 0.1, 1, 0): (1112.0, 3058.4, 4186.3), (4096, 0.1, 1, 1): (681.9, 1954.6, 2660.6),
    (8192, 0.0, 0, 0): (3415.7, 11207.1, 14681.4), (8192, 0.0, 0, 1): (1788.7, 6593.9, 8263.1), (8192, 0.1, 0, 0): (4244.1, 11320.8, 15619.1),
    (8192, 0.1, 0, 1): (2230.5, 5854.1, 8129.3), (8192, 0.0, 1, 0): (3411.3, 12037.3, 15479.7), (8192, 0.0, 1, 1): (1847.7, 7640.0, 9533.0),
    (8192, 0.1, 1, 0): (4215.3, 11619.2, 15894.8), (8192, 0.1, 1, 1): (2258.7, 6188.9, 8485.7),
}
REF_A100_LION_US = {(8192, "fp16"): 25.1, (8192, "bf16"): 25.0, (8192 ** 2, "fp16"): 651.9, (8192 ** 2, "bf16"): 710.1}


def bench_next(steps, warmup, settle):
    """What lies around the two headline kernels, timed with the same machinery. Attention: the reference's benchmark
    matrix (benchmarks/benchmark_flash_attention.py:195-209 and the table of fast_ops/flash_attention/README.md:76-175):
    [1, S, 12, 128] bf16 tensors through flash_attn, S in {2048, 4096, 8192}, causal or not, dropout 0 / 0.1, no bias / a
    [1, 1, 1, S] bias; forward (no autograd), backward alone (the two backward launches on saved O and LSE) and forward +
    backward through autograd. Lion: benchmarks/benchmark_lion.py:10-16 (one tensor of 8192 or 8192^2 elements, all-fp16
    or all-bf16, lr 1e-4, betas (0.9, 0.99), weight decay 0.1) and the 1.3 B-parameter set with all-bf16 tensors and with
    fp32 parameters + fp32 momentum."""
    import math

    import torch

    from fast_ops.lion.lion_optimizer import Lion
    from fast_ops_amd.flash_attention.flash_attention import attn_bwd_strided, attn_fwd_strided, flash_attn, next_dropout_state

    dev = "cuda:0"
    B, H, D = 1, 12, 128
    dims = (0, 2, 1, 3)
    rows = []
    g = torch.Generator().manual_seed(0)
    for S in (2048, 4096, 8192):
        q, k, v, go = (torch.randn(B, S, H, D, generator=g).to(torch.bfloat16).to(dev) for _ in range(4))
        bias_t = torch.randn(B, 1, 1, S, generator=g).to(torch.bfloat16).to(dev)
        for has_bias in (0, 1):
            for p_drop in (0.0, 0.1):
                for causal in (0, 1):
                    bias = bias_t if has_bias else None
                    flops = (2.0 if causal else 4.0) * B * H * S * S * D
                    f_step, f_kernel, f_min, _ = _time_steps(lambda: flash_attn(q, k, v, bias, bool(causal), p_drop), steps, warmup, settle,
                                                             wall_without_events=True)
                    drop = None if p_drop == 0.0 else (p_drop,) + next_dropout_state(B * H * S * S)
                    o, lse = attn_fwd_strided(q, k, v, dims, bool(causal), None, drop, bias)
                    b_step, b_kernel, b_min, _ = _time_steps(lambda: attn_bwd_strided(q, k, v, o, lse, go, dims, bool(causal), None, drop, bias),
                                                             steps, warmup, settle // 2, wall_without_events=True)
                    qr, kr, vr = (t.detach().requires_grad_(True) for t in (q, k, v))

                    def both():
                        flash_attn(qr, kr, vr, bias, bool(causal), p_drop).backward(go)
                        qr.grad = kr.grad = vr.grad = None

                    fb_step, fb_kernel, fb_min, _ = _time_steps(both, steps, warmup, settle // 2, wall_without_events=True)
                    ref = REF_A100_TRITON_US[(S, p_drop, has_bias, causal)]
                    rows.append({
                        "shape": f"({B},{H},{S},{D})", "dropout_p": p_drop, "bias": has_bias, "causal": causal,
                        "fwd_us": f_kernel * 1e3, "fwd_us_wall": f_step * 1e3, "fwd_tflops": flops / (f_kernel * 1e-3) / 1e12,
                        "bwd_us": b_kernel * 1e3, "bwd_us_wall": b_step * 1e3, "bwd_tflops": 2.5 * flops / (b_kernel * 1e-3) / 1e12,
                        "fwd_bwd_us": fb_kernel * 1e3, "fwd_bwd_us_wall": fb_step * 1e3,
                        "reference_a100_triton_us": {"fwd": ref[0], "bwd": ref[1], "fwd_bwd": ref[2]},
                    })
                    del o, lse, qr, kr, vr
        del q, k, v, go, bias_t
        torch.cuda.empty_cache()
    hp = dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)
    lion_rows = []
    for size in (8192, 8192 ** 2):
        for dt, name in ((torch.float16, "fp16"), (torch.bfloat16, "bf16")):
            prm = torch.nn.Parameter(torch.randn(size, generator=g).to(dt).to(dev))
            prm.grad = torch.randn(size, generator=g).to(dt).to(dev)
            opt = Lion([prm], **hp)
            l_step, l_kernel, l_min, _ = _time_steps(opt.step, steps, warmup, settle, wall_without_events=True)
            lion_rows.append({
                "elements": size, "dtypes": f"all {name}", "bytes_per_element": 10, "step_us": l_kernel * 1e3, "step_us_wall": l_step * 1e3,
                "gb_per_s": 10.0 * size / (l_kernel * 1e-3) / 1e9, "frac_of_hbm_peak": 10.0 * size / (l_kernel * 1e-3) / 1e9 / PEAK_HBM_GBS,
                "reference_a100_us": REF_A100_LION_US[(size, name)],
            })
            del opt, prm
    torch.cuda.empty_cache()
    n_params = sum(a * b for a, b in LION_LARGE_SHAPES)
    for p_dt, m_dt, name, nbytes in ((torch.bfloat16, torch.bfloat16, "all bf16", 10), (torch.float32, torch.float32, "fp32 parameters and gradients, fp32 momentum", 20),
                                     (torch.float32, torch.bfloat16, "fp32 parameters and gradients, bf16 momentum (the headline kernel)", 16)):
        params = [torch.nn.Parameter(torch.empty(sh, dtype=p_dt, device=dev).normal_(0, 0.02)) for sh in LION_LARGE_SHAPES]
        for prm in params:
            prm.grad = torch.empty_like(prm).normal_(0, 1e-2)
        opt = Lion(params, exp_avg_dtype=m_dt, **hp)
        l_step, l_kernel, l_min, _ = _time_steps(opt.step, min(steps, 50), warmup, min(settle, 20))
        lion_rows.append({
            "elements": n_params, "dtypes": name, "bytes_per_element": nbytes, "step_us": l_kernel * 1e3, "step_us_wall": l_step * 1e3,
            "gb_per_s": float(nbytes) * n_params / (l_kernel * 1e-3) / 1e9, "frac_of_hbm_peak": float(nbytes) * n_params / (l_kernel * 1e-3) / 1e9 / PEAK_HBM_GBS,
        })
        del opt, params
        torch.cuda.empty_cache()
    return {"path": "next", "attention_reference_matrix": rows, "lion": lion_rows,
            "note": "times from HIP events around each call (mean over the timed steps); *_wall = host wall clock per call over as many calls "
                    "without events; reference figures are the reference's own published A100 timings, quoted for context"}


def bench_clock(steps, warmup, settle):
    """What the chip's clock does under this kernel: the 256-row attention kernel with 32 ... 512 workgroups (one per CU up
    to 256, so the launch time is one workgroup's time), the headline shape on random and on all-zero operands, and the
    vendor library's GEMM on both. Run under `rocprofv3 --pmc GRBM_GUI_ACTIVE --kernel-trace`, the counter divided by a
    kernel's duration is the clock it ran at."""
    import torch

    from fast_ops.flash_attention.flash_attention import multi_head_attention
    from fast_ops_amd import _lib

    dev, S, D = "cuda:0", 8192, 128
    scale = 1.0 / (D ** 0.5)
    out = {"busy_cus": [], "operands": [], "gemm": []}
    (q, k, v), g = _attn_inputs(2, 16, S, D, torch.bfloat16, dev)
    _lib.tune_set("attn.variant", _lib.FO_ATTN_KERNEL_ROWS256_W8)
    try:
        for heads in (2, 4, 8, 12, 16, 32):
            qq, kk, vv = (t.view(32, S, D)[:heads].view(1, heads, S, D) for t in (q, k, v))
            _, ms, ms_min, _ = _time_steps(lambda: multi_head_attention(qq, kk, vv, causal=True, softmax_scale=scale), steps, warmup, settle)
            wgs = heads * 16
            out["busy_cus"].append({"heads": heads, "workgroups": wgs, "kernel_ms_avg": ms, "kernel_ms_min": ms_min,
                                    "tflops": 2.0 * heads * S * S * D / (ms * 1e-3) / 1e12})
        for name, make in (("standard normal", lambda t: t), ("all zero", torch.zeros_like), ("all one", torch.ones_like)):
            qq, kk, vv = make(q), make(k), make(v)
            _, ms, ms_min, _ = _time_steps(lambda: multi_head_attention(qq, kk, vv, causal=True, softmax_scale=scale), steps, warmup, settle)
            out["operands"].append({"operands": name, "kernel_ms_avg": ms, "kernel_ms_min": ms_min, "tflops": 2.0 * 32 * S * S * D / (ms * 1e-3) / 1e12})
    finally:
        _lib.tune_set("attn.variant", -1)
    n = 8192
    a, b = (torch.randn(n, n, generator=g).to(torch.bfloat16).to(dev) for _ in range(2))
    for name, make in (("standard normal", lambda t: t), ("all zero", torch.zeros_like)):
        aa, bb = make(a), make(b)
        _, ms, ms_min, _ = _time_steps(lambda: torch.matmul(aa, bb), steps, warmup, settle)
        out["gemm"].append({"operands": name, "kernel_ms_avg": ms, "kernel_ms_min": ms_min, "tflops": 2.0 * n ** 3 / (ms * 1e-3) / 1e12})
    return out


def bench_power(seconds):
    """Socket power while each kernel runs back to back for `seconds`: the attention forward of the headline shape on
    standard-normal and on all-zero operands, its backward, the vendor library's GEMM on both kinds of operands, and the
    fused Lion step. Power is the amdgpu driver's own sensor (hwmon power1_input or power1_average of the card, in
    microwatts), read every 10 ms by a host thread; a kernel's figure is the mean over its loop without the first second.
    Beside it the time per launch over the same loop, by events."""
    import glob
    import threading

    import torch

    from fast_ops.flash_attention.flash_attention import multi_head_attention
    from fast_ops_amd.flash_attention.flash_attention import attn_bwd_strided, attn_fwd_strided

    sensors = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")) or \
        sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average"))
    if not sensors:
        print("bench.py --path power: no power sensor under /sys/class/drm/card*/device/hwmon", file=sys.stderr)
        sys.exit(2)
    sensor = sensors[0]
    samples, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            try:
                samples.append((time.perf_counter(), int(open(sensor).read()) * 1e-6))
            except (OSError, ValueError):
                pass
            time.sleep(0.01)

    th = threading.Thread(target=sampler, daemon=True)
    th.start()
    dev, B, H, S, D = "cuda:0", 2, 16, 8192, 128
    scale = 1.0 / (D ** 0.5)
    (q, k, v), g = _attn_inputs(B, H, S, D, torch.bfloat16, dev)
    go = torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(dev)
    o, lse = attn_fwd_strided(q, k, v, (0, 1, 2, 3), True, scale)
    zq = torch.zeros_like(q)
    n = 8192
    a, b = (torch.randn(n, n, generator=g).to(torch.bfloat16).to(dev) for _ in range(2))
    za = torch.zeros_like(a)
    _params, opt = _lion_setup(LION_LARGE_SHAPES, dev)
    cases = [
        ("attention forward, standard-normal operands", lambda: multi_head_attention(q, k, v, causal=True, softmax_scale=scale), 2.0 * B * H * S * S * D),
        ("attention forward, all-zero operands", lambda: multi_head_attention(zq, zq, zq, causal=True, softmax_scale=scale), 2.0 * B * H * S * S * D),
        ("attention backward, standard-normal operands", lambda: attn_bwd_strided(q, k, v, o, lse, go, (0, 1, 2, 3), True, scale), 5.0 * B * H * S * S * D),
        ("library GEMM 8192^3 bf16, standard-normal operands", lambda: torch.matmul(a, b), 2.0 * n ** 3),
        ("library GEMM 8192^3 bf16, all-zero operands", lambda: torch.matmul(za, za), 2.0 * n ** 3),
        ("fused Lion step, 1.3 B parameters", lambda: opt.step(), None),
    ]
    torch.cuda.synchronize()
    time.sleep(1.0)
    t_idle_end = time.perf_counter()
    out = {"sensor": sensor, "seconds_per_kernel": seconds, "kernels": []}
    for name, step, flops in cases:
        for _ in range(5):
            step()
        torch.cuda.synchronize()
        e0, e1 = _events(2)
        t0 = time.perf_counter()
        launches = 0
        e0.record()
        while time.perf_counter() - t0 < seconds:
            for _ in range(20):
                step()
            launches += 20
            torch.cuda.synchronize()
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        watts = [w for t, w in samples if t0 + min(1.0, seconds / 2) <= t <= t1]
        ms = e0.elapsed_time(e1) / launches
        row = {"kernel": name, "launches": launches, "ms_per_launch": ms, "socket_watts_mean": sum(watts) / max(len(watts), 1),
               "socket_watts_max": max(watts) if watts else None, "samples": len(watts)}
        if flops is not None:
            row["tflops"] = flops / (ms * 1e-3) / 1e12
        out["kernels"].append(row)
        time.sleep(0.5)
    stop.set()
    th.join()
    idle = [w for t, w in samples if t <= t_idle_end]
    out["socket_watts_idle"] = sum(idle) / max(len(idle), 1)
    return out


def bench_ablations(steps, warmup, settle):
    """Timing ablations of the 256-row attention kernel at the headline shape: what each part of the kernel costs in
    cycles and in clock. Needs a library built with `python -m fast_ops_amd.build --ablations` (the variants leave work
    out and produce wrong results by design; a default build does not contain them). Under
    `rocprofv3 --pmc GRBM_GUI_ACTIVE SQ_VALU_MFMA_BUSY_CYCLES --kernel-trace` every variant is a kernel of its own name."""
    import torch

    from fast_ops.flash_attention.flash_attention import multi_head_attention
    from fast_ops_amd import _lib

    if _lib.load().fo_tune_get(b"build.ablations") != 1:
        print("bench.py --path ablations needs a library built with `python -m fast_ops_amd.build --ablations`", file=sys.stderr)
        sys.exit(2)
    B, H, S, D = 2, 16, 8192, 128
    (q, k, v), _ = _attn_inputs(B, H, S, D, torch.bfloat16, "cuda:0")
    scale = 1.0 / (D ** 0.5)
    names = {16: "full kernel (eight waves x 32 rows)", 257: "no global->LDS copies", 258: "no exponentials (and no scale-and-shift)",
             260: "no LDS fragment reads", 263: "none of the three", 320: "no barrier", 32: "four waves x 64 rows", 0: "128-row kernel"}
    out = []
    try:
        for causal, variants in ((False, (16, 257, 258, 260, 263, 320, 32)), (True, (16, 32, 0))):
            flops = (2.0 if causal else 4.0) * B * H * S * S * D
            for var in variants:
                _lib.tune_set("attn.variant", var)
                _, ms, ms_min, _ = _time_steps(lambda: multi_head_attention(q, k, v, causal=causal, softmax_scale=scale), steps, warmup, settle)
                out.append({"causal": causal, "variant": var, "what": names[var], "kernel_ms_avg": ms, "kernel_ms_min": ms_min, "tflops_equivalent": flops / (ms * 1e-3) / 1e12})
    finally:
        _lib.tune_set("attn.variant", -1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--settle", type=int, default=100,
                    help="clock-settle launches ahead of the warm-up of every timed section, in blocks of this many until two blocks in a row "
                         "agree within 1.5 %% and a second has passed (reported, not counted as warm-up)")
    ap.add_argument("--path", choices=["both", "attn", "lion", "next", "copy", "clock", "power", "ablations"], default="both",
                    help="next: the reference's benchmark matrix (forward, backward, forward+backward with bias and dropout) and the "
                         "typed Lion kernels; copy: a plain 4 GiB device copy, the known-size reference that HBM byte counters are scaled by; "
                         "clock: the attention kernel against the number of busy CUs and the operand bits, with the library GEMM; "
                         "power: socket power (the driver's sensor) while each kernel loops for 3 s; "
                         "ablations: the attention kernel with parts left out (needs a build with --ablations)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the two headline kernels (no backward, library GEMM or other configurations): for profiler runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: both kernels are single-device and this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    from fast_ops_amd import _lib

    _lib.load()   # fail loudly when the HIP library is missing
    if args.path == "copy":
        n = 1 << 30
        src = torch.ones(n, dtype=torch.float32, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(args.warmup + args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": 4 * n, "copy_bytes_written": 4 * n, "launches": args.warmup + args.steps}))
        return
    if args.path == "clock":
        print(json.dumps(bench_clock(args.steps, args.warmup, args.settle)))
        return
    if args.path == "next":
        print(json.dumps(bench_next(args.steps, args.warmup, args.settle)))
        return
    if args.path == "power":
        print(json.dumps({"path": "power", **bench_power(3.0)}))
        return
    if args.path == "ablations":
        print(json.dumps(bench_ablations(args.steps, args.warmup, args.settle)))
        return
    cpu = not args.no_cpu_baseline
    extras = not args.headline_only
    attn = bench_attention(args.steps, args.warmup, args.settle, cpu, extras) if args.path in ("both", "attn") else None
    lion = bench_lion(args.steps, args.warmup, args.settle, cpu, extras) if args.path in ("both", "lion") else None
    head = attn if attn is not None else lion
    line = {
        "metric": "FA fwd TFLOP/s (bf16, S=8K D=128 causal) + fused Lion HBM GB/s",
        "value": head["value"],
        "unit": "TFLOP/s" if attn is not None else "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if attn is not None else "f32",
        "data": "synthetic",
        "config": {"workload": head["workload"] + ("; second path: " + lion["workload"] if attn is not None and lion is not None else "")},
        "roofline": head["roofline"],
        "settle": head["settle"],
    }
    if "cpu_baseline" in head:
        line["cpu_baseline"] = head["cpu_baseline"]
    if attn is not None and lion is not None:
        line["lion"] = {k: v for k, v in lion.items() if k not in ("workload", "configs")}
    if attn is not None and "bwd" in attn:
        line["attn_bwd"] = attn["bwd"]
    if attn is not None and "library_gemm" in attn:
        line["library_gemm"] = attn["library_gemm"]
    if attn is not None and "headline_variants" in attn:
        line["headline_variants"] = attn["headline_variants"]
    configs = {}
    for part in (attn, lion):
        if part is not None:
            configs.update(part.get("configs", {}))
    if configs:
        line["configs"] = configs
    print(json.dumps(line))


if __name__ == "__main__":
    main()

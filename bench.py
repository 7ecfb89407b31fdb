"""Benchmark of the two hot paths on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--path both|attn|lion] [--no-cpu-baseline]

Prints ONE JSON line. The headline value is the attention forward throughput at B=2 H=16 S=8192 D=128 bf16 causal
(FLOPs counted as 2*B*H*S^2*D); the fused Lion step over 1,308,622,848 fp32 parameters with bf16 momentum (16 bytes
per parameter) is reported in the "lion" object of the same line, each with its roofline and a CPU baseline timed on
this host's cores. The attention backward of the same shape is reported in "attn_bwd", and the rate of the vendor
library's plain bf16 GEMM on random operands on the same box in "library_gemm" (what MFMA code reaches here at all).
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


def _measured_traffic(key):
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this workload (the runs and the
    scaling against a plain copy are in profiles/hbm_traffic_pmc_*.txt); None when that file is absent."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            return json.load(f).get(key)
    except OSError:
        return None


def _events(n):
    import torch

    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _time_steps(step, steps, warmup):
    """W untimed steps, then K timed steps bracketed by synchronize; per-launch durations from HIP events recorded on
    the stream the kernels are launched on (torch's current stream)."""
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    ev = _events(steps + 1)
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        step()
        ev[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per_launch = [ev[i].elapsed_time(ev[i + 1]) for i in range(steps)]
    return wall_ms / steps, sum(per_launch) / steps, min(per_launch)


def bench_attention(steps, warmup, cpu_baseline):
    import torch

    from fast_ops.flash_attention.flash_attention import multi_head_attention

    B, H, S, D = 2, 16, 8192, 128
    dev = "cuda:0"
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(dev) for _ in range(3))
    scale = 1.0 / (D ** 0.5)
    flops = 2.0 * B * H * S * S * D      # causal-halved 4*B*H*S^2*D
    out = {}

    def step():
        out["o"], out["lse"] = multi_head_attention(q, k, v, causal=True, softmax_scale=scale, return_lse=True)

    ms_step, ms_kernel, ms_min = _time_steps(step, steps, warmup)
    res = {
        "value": flops / (ms_step * 1e-3) / 1e12,
        "ms_per_step": ms_step,
        "roofline": {
            "bound": "mfma", "achieved": flops / (ms_kernel * 1e-3) / 1e12, "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s",
            "frac": flops / (ms_kernel * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "traffic": _measured_traffic("attn"),
            "kernel_ms_avg": ms_kernel, "kernel_ms_min": ms_min, "flops_per_launch": flops,
        },
        "workload": f"attention fwd B={B} H={H} S={S} D={D} bf16 causal, scale 1/sqrt({D})",
    }
    # the backward of the same workload (dQ, dK, dV; two launches), reported beside the headline, not part of it
    from fast_ops_amd.flash_attention.flash_attention import attn_bwd_strided

    go = torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(dev)
    o_fix, lse_fix = out["o"], out["lse"]
    bwd_flops = 5.0 * B * H * S * S * D      # causal-halved 10*B*H*S^2*D (five GEMMs; the kernels recompute two more)
    b_step, b_kernel, b_min = _time_steps(lambda: attn_bwd_strided(q, k, v, o_fix, lse_fix, go, (0, 1, 2, 3), True, scale), steps, warmup)
    res["bwd"] = {
        "value": bwd_flops / (b_step * 1e-3) / 1e12, "unit": "TFLOP/s", "ms_per_step": b_step,
        "roofline": {"bound": "mfma", "achieved": bwd_flops / (b_kernel * 1e-3) / 1e12, "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": bwd_flops / (b_kernel * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS, "traffic": None,
                     "kernel_ms_avg": b_kernel, "kernel_ms_min": b_min, "flops_per_launch": bwd_flops},
        "workload": "attention bwd (dQ + dK/dV kernels) of the same shape, FLOPs by the five-GEMM count",
    }
    # yardstick, not part of the headline: the vendor library's plain bf16 GEMM on the same box with the same kind of
    # data. Under a full-chip MFMA load the clock follows the power drawn, which depends on the operand bits (all-zero
    # operands run a third faster than random ones), so the published peak is not what random data can reach.
    n = 8192
    ga, gb = (torch.randn(n, n, generator=g).to(torch.bfloat16).to(dev) for _ in range(2))
    _, g_kernel, _ = _time_steps(lambda: torch.matmul(ga, gb), 20, 20)
    res["library_gemm"] = {
        "value": 2.0 * n ** 3 / (g_kernel * 1e-3) / 1e12, "unit": "TFLOP/s", "frac_of_peak": 2.0 * n ** 3 / (g_kernel * 1e-3) / 1e12 / PEAK_MFMA_TFLOPS,
        "what": f"torch.matmul (hipBLASLt) bf16 {n}x{n}x{n}, standard normal operands, same box, timed after the attention runs",
    }
    del ga, gb
    if cpu_baseline:
        # bounded sample: all (batch, head) slices of the same workload through the oracle's fp32 vanilla path on all host
        # cores, stopped after about 15 s; the rate is that of the slices that were finished
        from oracle.attention_oracle import attention_fwd_oracle

        torch.set_num_threads(os.cpu_count())
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
            "value": n_sl * 2.0 * S * S * D / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{n_sl} of {B * H} (batch, head) slices of the same shape, fp32 vanilla softmax(QK^T)V on the host, {dt:.2f} s",
        }
    return res


def bench_lion(steps, warmup, cpu_baseline):
    import torch

    from fast_ops.lion.lion_optimizer import Lion

    dev = "cuda:0"
    shapes = [(2048, 8192)] * 39 + [(8192, 2048)] * 39
    n_params = sum(a * b for a, b in shapes)
    gen = torch.Generator(device=dev).manual_seed(0)
    params = [torch.nn.Parameter(torch.randn(s, device=dev, generator=gen) * 0.02) for s in shapes]
    hp = dict(lr=1e-4, betas=(0.9, 0.99), weight_decay=0.1)
    opt = Lion(params, **hp)
    for p in params:
        opt.state[p]["exp_avg"] = (torch.randn(p.shape, device=dev, generator=gen) * 1e-3).to(torch.bfloat16)
        p.grad = torch.randn(p.shape, device=dev, generator=gen) * 1e-2
    nbytes = 16.0 * n_params
    ms_step, ms_kernel, ms_min = _time_steps(opt.step, steps, warmup)
    res = {
        "value": nbytes / (ms_step * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": ms_step, "dtype": "f32 params/grads, bf16 momentum",
        "roofline": {
            "bound": "hbm", "achieved": nbytes / (ms_kernel * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": nbytes / (ms_kernel * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": _measured_traffic("lion"),
            "kernel_ms_avg": ms_kernel, "kernel_ms_min": ms_min, "bytes_per_launch": nbytes,
        },
        "workload": f"fused Lion step, {len(shapes)} tensors (39 x 2048x8192 + 39 x 8192x2048) = {n_params} fp32 params, bf16 momentum",
    }
    if cpu_baseline:
        # bounded sample: 8 of the 78 tensors (134,217,728 parameters) through the four reference statements on all host
        # cores, 3 steps
        from oracle.lion_oracle import lion_step_torch

        torch.set_num_threads(os.cpu_count())
        n_t = 8
        ps = [params[i].detach().cpu().clone() for i in range(n_t)]
        gs = [params[i].grad.cpu().clone() for i in range(n_t)]
        ms = [opt.state[params[i]]["exp_avg"].cpu().clone() for i in range(n_t)]
        lion_step_torch(ps, gs, ms, hp["lr"], hp["betas"], hp["weight_decay"])     # warm-up
        reps = 3
        t0 = time.perf_counter()
        for _ in range(reps):
            lion_step_torch(ps, gs, ms, hp["lr"], hp["betas"], hp["weight_decay"])
        dt = (time.perf_counter() - t0) / reps
        n_el = sum(p.numel() for p in ps)
        res["cpu_baseline"] = {
            "value": 16.0 * n_el / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{n_t} of 78 tensors ({n_el} parameters), vanilla 4-statement PyTorch Lion step on the host, {dt * 1e3:.1f} ms per step, {reps} steps",
        }
    del opt, params
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults: the GPU's clocks take a few dozen launches to settle after idling (per-launch time of the attention
    # kernel wanders by 25 % over the first 30 launches, then stays within 1 %), so the warm-up is longer than usual
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--path", choices=["both", "attn", "lion", "copy"], default="both",
                    help="copy: a plain 4 GiB device copy, the known-size reference that HBM byte counters are scaled by")
    ap.add_argument("--no-cpu-baseline", action="store_true")
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
    cpu = not args.no_cpu_baseline
    attn = bench_attention(args.steps, args.warmup, cpu) if args.path in ("both", "attn") else None
    lion = bench_lion(args.steps, args.warmup, cpu) if args.path in ("both", "lion") else None
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
    }
    if "cpu_baseline" in head:
        line["cpu_baseline"] = head["cpu_baseline"]
    if attn is not None and lion is not None:
        line["lion"] = {k: v for k, v in lion.items() if k != "workload"}
    if attn is not None and "bwd" in attn:
        line["attn_bwd"] = attn["bwd"]
    if attn is not None and "library_gemm" in attn:
        line["library_gemm"] = attn["library_gemm"]
    print(json.dumps(line))


if __name__ == "__main__":
    main()

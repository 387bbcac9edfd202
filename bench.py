"""Headline benchmark: logbmm forward + backward, fp32, B=64, M=K=N=512, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one forward and one backward of the hot path through the C ABI on inputs
already resident in HBM (seeded synthetic log-potentials).  Prints one JSON line:
semiring GOP/s (6*B*M*K*N semiring operations per step), the roofline of the dominant
kernel measured with events around its launches, and the reference's CPU formulation
(the torch broadcast) timed on this host's cores on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

B, M, K, N = 64, 512, 512, 512
FP32_VALU_PEAK_TFLOPS = 157.3  # MI355X FP32 peak (vector with packed FMA = fp32 matrix cores)
BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak
# HBM bytes per launch of the dominant kernel (k_log_bwd_split_both): rocprofv3 --pmc
# FETCH_SIZE + WRITE_SIZE in KiB per dispatch, scale factor 1.00 against a known-size copy in
# the same run; the two figures are those of profiles/logbmm_headline_B64_512.md.
DOMINANT_FETCH_KIB, DOMINANT_WRITE_KIB = 242399, 131072
DOMINANT_TRAFFIC_BYTES = (DOMINANT_FETCH_KIB + DOMINANT_WRITE_KIB) * 1024


def cpu_baseline(torch, sample_batches=64):
    """The reference's CPU formulation (README.md:31-35): broadcast add + logsumexp, and
    autograd backward, on `sample_batches` items of the headline shape, one item per
    chunk (a 512 MB fp32 intermediate each)."""
    import oracle

    # the threads torch's CPU kernels run on: OMP_NUM_THREADS where the host sets it, else the
    # cores this process may be scheduled on
    cores = torch.get_num_threads()
    if "OMP_NUM_THREADS" not in os.environ and hasattr(os, "sched_getaffinity"):
        cores = len(os.sched_getaffinity(0))
        torch.set_num_threads(cores)
    torch.manual_seed(0)
    a = torch.randn(sample_batches, M, K)
    b = torch.randn(sample_batches, K, N)
    g = torch.randn(sample_batches, M, N)

    def one(i):
        ai = a[i:i + 1].clone().requires_grad_(True)
        bi = b[i:i + 1].clone().requires_grad_(True)
        out = oracle.logbmm_broadcast(ai, bi)
        out.backward(g[i:i + 1])
        return ai.grad, bi.grad

    one(0)  # warm-up
    t0 = time.perf_counter()
    for i in range(sample_batches):
        one(i)
    dt = time.perf_counter() - t0
    ops = 6.0 * sample_batches * M * K * N
    return {
        "value": round(ops / dt / 1e9, 3),
        "unit": "semiring GOP/s",
        "cores": cores,
        "kind": "port",
        "sample": "%d of the %d batch items of the headline shape, one item per chunk, torch broadcast "
                  "logsumexp fwd + autograd bwd, %.1f s" % (sample_batches, B, dt),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true", help="skip the float64 check of all items before timing")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU only; every batch item is independent, so more GPUs "
                 "would shard the batch axis with no exchange. Run with --gpus 1.")

    import torch

    from genbmm_amd import _lib

    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    a = torch.randn(B, M, K).to(dev)
    b = torch.randn(B, K, N).to(dev)
    g = torch.randn(B, M, N).to(dev)
    out = torch.empty(B, M, N, device=dev)
    ga, gb = torch.empty_like(a), torch.empty_like(b)
    stats = torch.empty(lib.genbmm_logbmm_stats_size(B, M, K, N), device=dev)
    stream = _lib.stream_of(a)
    p = _lib.ptr
    null = p(None)

    def fwd():
        _lib.check(lib.genbmm_logbmm_fwd(p(a), p(b), p(out), p(stats), B, M, K, N, stream), "fwd")

    def bwd():  # both gradients in one call, like the reference's _genbmm.backward
        _lib.check(lib.genbmm_logbmm_bwd(p(a), p(b), p(out), p(g), p(stats), p(ga), p(gb), B, M, K, N, stream), "bwd")

    # Before anything is timed: the buffers the timed steps write are checked, every batch item,
    # against float64 torch on the device (the broadcast form of README.md:31-35 and its autograd
    # gradients, an item at a time - 1 GB of float64 terms each).  A wrong kernel ends the run here.
    checked = None
    if not args.no_verify:
        fwd(); bwd()
        worst = [0.0, 0.0, 0.0]
        for i in range(B):
            a64, b64 = a[i].double().requires_grad_(True), b[i].double().requires_grad_(True)
            ref = torch.logsumexp(a64[:, :, None] + b64[None, :, :], dim=1)
            ra, rb = torch.autograd.grad(ref, (a64, b64), g[i].double())
            for j, (got, want) in enumerate(((out[i], ref.detach()), (ga[i], ra), (gb[i], rb))):
                err = float(((got.double() - want).abs() / (1e-5 + 1e-5 * want.abs())).max())
                worst[j] = max(worst[j], err)
            del a64, b64, ref, ra, rb
        if not max(worst) <= 1.0:
            sys.exit("bench.py: results differ from float64 beyond rtol 1e-5 + atol 1e-5 (out, grad_a, grad_b: "
                     "%s x the tolerance)" % worst)
        checked = {"items": B, "reference": "float64 torch broadcast logsumexp + autograd on the device",
                   "rtol": 1e-5, "atol": 1e-5,
                   "worst_error_over_tolerance": {"out": round(worst[0], 4), "grad_a": round(worst[1], 4),
                                                  "grad_b": round(worst[2], 4)}}

    for _ in range(args.warmup):
        fwd(); bwd()
    torch.cuda.synchronize()
    # a plain elementwise kernel of known size (B*M*K*4 bytes read, the same written; float add,
    # the only one in this program): the yardstick the FETCH_SIZE / WRITE_SIZE counters are scaled
    # by in profiles/
    calib = torch.add(a, 1.0)
    del calib

    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.steps):
        ev[s][0].record(); fwd()
        ev[s][1].record(); bwd()
        ev[s][2].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0

    ms_fwd = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    ms_bwd = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps
    # The same events, first and last five timed steps apart: after any idle period (the host-side
    # set-up above is one) this GPU runs its first ~25 ms of work slower and then settles, whatever
    # the kernel - a short run (few warm-up steps) is timed inside that window, a long one past it.
    head, tail = ev[:5], ev[-5:]

    def mean(pairs):
        return round(sum(x.elapsed_time(y) for x, y in pairs) / len(pairs), 4)

    trend = {
        "ms_step_first5": mean([(e[0], e[2]) for e in head]), "ms_step_last5": mean([(e[0], e[2]) for e in tail]),
        "ms_fwd_first5": mean([(e[0], e[1]) for e in head]), "ms_fwd_last5": mean([(e[0], e[1]) for e in tail]),
        "ms_bwd_first5": mean([(e[1], e[2]) for e in head]), "ms_bwd_last5": mean([(e[1], e[2]) for e in tail]),
    }
    # and, outside the timed region and of no influence on `value`: the step time once settled
    # (60 more steps straight behind the timed ones, the last 20 of them averaged)
    more = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(60)]
    for e in more:
        e[0].record(); fwd()
        e[1].record(); bwd()
        e[2].record()
    torch.cuda.synchronize()
    trend["ms_step_settled"] = round(more[40][0].elapsed_time(more[59][2]) / 20, 4)
    trend["ms_bwd_settled"] = mean([(e[1], e[2]) for e in more[40:]])
    ms_step = dt * 1e3 / args.steps
    bmkn = float(B) * M * K * N
    value = 6.0 * bmkn / (ms_step * 1e-3) / 1e9

    # dominant kernel = the backward launch, which computes both gradients (algorithmic 4*BMKN
    # flops = two multiply-adds per (b,m,k,n)); its event-bracketed time includes the 4 us
    # fix-up launch behind it.  The products have fp32 accuracy, but the kernel takes each as six
    # bf16 partial products on v_mfma_f32_32x32x16_bf16 (every factor in three bf16 parts that add
    # up to it exactly), so the roofline that bounds it is the bf16 matrix pipe at one sixth of its
    # rate: peak = 2500 / 6 TFLOP/s of algorithmic flops.  The same rate against the fp32 matrix /
    # vector peak (157.3, what the fp32 instruction could reach at best) is reported beside it.
    ms_dom = ms_bwd
    achieved = 4.0 * bmkn / (ms_dom * 1e-3) / 1e12
    peak = BF16_MFMA_PEAK_TFLOPS / 6.0
    roofline = {
        "bound": "mfma",
        "kernel": "k_log_bwd_split_both (grad_a and grad_b tiles in one launch, operands formed again "
                  "from a, b, out and the maxima, each cut into three bf16 parts; six bf16 matrix "
                  "instructions per fp32-accurate product block)",
        "achieved": round(achieved, 3),
        "peak": round(peak, 1),
        "unit": "TFLOP/s",
        "frac": round(achieved / peak, 4),
        "traffic": DOMINANT_TRAFFIC_BYTES,
        "avg_launch_ms": round(ms_dom, 4),
        "peak_is": "MI355X dense bf16 matrix peak 2500 TFLOP/s / 6 bf16 products per fp32-accurate product",
        "executed_bf16_tflops": round(6.0 * achieved, 1),
        "frac_of_fp32_peak_157.3": round(achieved / FP32_VALU_PEAK_TFLOPS, 4),
    }

    # end-to-end through the public autograd API (allocations included), for the record
    import genbmm_amd as genbmm

    ar, br = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    for _ in range(2):
        genbmm.logbmm(ar, br).backward(g)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(args.steps):
        ar.grad = br.grad = None
        genbmm.logbmm(ar, br).backward(g)
    torch.cuda.synchronize()
    ms_autograd = (time.perf_counter() - t1) * 1e3 / args.steps

    line = {
        "metric": "semiring GOP/s logbmm fwd+bwd fp32 B=64 512^3; % FP32 VALU peak",
        "value": round(value, 1),
        "unit": "semiring GOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "logbmm fwd+bwd, a,b,g ~ Normal(0,1) seed 0, B=64 M=K=N=512 (headline)",
                   "B": B, "M": M, "K": K, "N": N, "ops_per_step": 6.0 * bmkn},
        "pct_fp32_valu_peak": round(100.0 * value / 1e3 / FP32_VALU_PEAK_TFLOPS, 3),
        "ms_fwd": round(ms_fwd, 4),
        "ms_bwd": round(ms_bwd, 4),
        "step_time_trend": trend,
        "verified_before_timing": checked,
        "ms_per_step_autograd_api": round(ms_autograd, 4),
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline(torch),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

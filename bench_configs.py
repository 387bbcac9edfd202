"""Timing of every benchmark configuration (BASELINE.json) on one MI355X (bench.py covers only the
headline line the driver reads).

    python bench_configs.py [--reps 20] [--cpu]

For each configuration: median device time of the C-ABI calls on pre-allocated outputs
(HIP events on torch's current stream, 5 warm-ups), semiring GOP/s and % of the FP32
vector peak (157.3 TFLOP/s) from the algorithmic operation count, and HBM GB/s from the
algorithmic byte count.  --cpu adds the reference's CPU formulation (torch broadcast) for
configuration 0.  One JSON object per line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import torch  # noqa: E402

from genbmm_amd import _lib  # noqa: E402

PEAK_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def timed(fn, reps):
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        ts.append(e0.elapsed_time(e1))
    ts.sort()
    return ts[len(ts) // 2]


def report(name, ms, ops, nbytes, extra=None):
    line = {
        "config": name,
        "ms": round(ms, 4),
        "semiring_GOPs": round(ops / ms / 1e6, 1),
        "pct_fp32_vector_peak": round(100 * ops / (ms * 1e-3) / (PEAK_TFLOPS * 1e12), 2),
        "algorithmic_GBs": round(nbytes / ms / 1e6, 1),
        "pct_hbm_peak": round(100 * nbytes / (ms * 1e-3) / (PEAK_HBM_GBS * 1e9), 2),
    }
    if extra:
        line.update(extra)
    print(json.dumps(line), flush=True)


def dense_log(lib, dev, B, M, K, N, reps, name, dist="randn", path=0, graph=False, dtype=torch.float32, pad=None):
    """dtype float16 / bfloat16: the `_f16` / `_bf16` entry points on tensors of that type (and, for
    comparison, the float entry points with the widening and narrowing copies around them).
    pad = (value, rows): the last `rows` rows of every a hold `value` (padding), no gradient flows into them."""
    torch.manual_seed(0)
    mk = torch.randn if dist == "randn" else torch.rand
    a, b = mk(B, M, K).to(dev).to(dtype), mk(B, K, N).to(dev).to(dtype)
    g = (torch.ones(B, M, N) if dist == "rand" else torch.randn(B, M, N)).to(dev).to(dtype)
    if pad is not None:
        a[:, M - pad[1]:, :] = pad[0]
        g[:, M - pad[1]:, :] = 0
    out, ga, gb = torch.empty(B, M, N, device=dev, dtype=dtype), torch.empty_like(a), torch.empty_like(b)
    stats = torch.empty(lib.genbmm_logbmm_stats_size_path(B, M, K, N, path), device=dev)
    s, p = _lib.stream_of(a), _lib.ptr
    sfx = _lib.HALF_SUFFIX.get(dtype, "")
    fwd, bwd = getattr(lib, "genbmm_logbmm_fwd_path" + sfx), getattr(lib, "genbmm_logbmm_bwd_path" + sfx)

    def f():
        _lib.check(fwd(p(a), p(b), p(out), p(stats), B, M, K, N, path, s), "fwd")

    def bw():
        _lib.check(bwd(p(a), p(b), p(out), p(g), p(stats), p(ga), p(gb), B, M, K, N, path, s), "bwd")

    def step():
        f()
        bw()

    ms, mf, mb = timed(step, reps), timed(f, reps), timed(bw, reps)
    extra_graph = {}
    if graph:  # the same step captured once into a HIP graph and replayed (launch-bound shapes)
        gr, cap = torch.cuda.CUDAGraph(), torch.cuda.Stream()
        cap.wait_stream(torch.cuda.current_stream())
        with torch.cuda.graph(gr, stream=cap):
            s = _lib.stream_of(a)
            step()
        s = _lib.stream_of(a)
        extra_graph = {"ms_graph_replay": round(timed(gr.replay, reps), 4)}
    if sfx:  # the same step through the float kernels: widen a, b, g; narrow out and the gradients
        o32, ga32, gb32 = torch.empty(B, M, N, device=dev), torch.empty(B, M, K, device=dev), torch.empty(B, K, N, device=dev)

        def widened():
            x, y = a.float(), b.float()
            _lib.check(lib.genbmm_logbmm_fwd_path(p(x), p(y), p(o32), p(stats), B, M, K, N, path, s), "fwd")
            o = o32.to(dtype)
            gg = g.float()
            _lib.check(lib.genbmm_logbmm_bwd_path(p(x), p(y), p(o32), p(gg), p(stats), p(ga32), p(gb32), B, M, K, N, path, s), "bwd")
            return o, ga32.to(dtype), gb32.to(dtype)

        extra_graph["ms_float_kernels_with_casts"] = round(timed(widened, reps), 4)
    bmkn = float(B) * M * K * N
    nbytes = float(a.element_size()) * B * (3 * M * K + 3 * K * N + 3 * M * N)
    report(name, ms, 6 * bmkn, nbytes, {"path": {0: "factored (bf16 matrix instruction on three-part factors where the shape is made of full tiles)", 1: "online-exact", 2: "factored-valu", 3: "factored, factors kept (fp32 matrix instruction)", 4: "factored, fp32 matrix instruction"}[path],
                                        "workspace_MB": round(stats.numel() * 4 / 1e6, 2),
                                        "ms_fwd": round(mf, 4), "ms_bwd": round(mb, 4), **extra_graph})


def dense_log2(lib, dev, B, M, K, N, reps):
    """The second-order terms of logbmm (both cotangents given): one library call."""
    torch.manual_seed(0)
    a, b, g = torch.randn(B, M, K).to(dev), torch.randn(B, K, N).to(dev), torch.randn(B, M, N).to(dev)
    ua, ub = torch.randn(B, M, K).to(dev), torch.randn(B, K, N).to(dev)
    out = torch.empty(B, M, N, device=dev)
    stats = torch.empty(lib.genbmm_logbmm_stats_size(B, M, K, N), device=dev)
    ga, gb, gg = torch.empty_like(a), torch.empty_like(b), torch.empty_like(g)
    s, p = _lib.stream_of(a), _lib.ptr
    _lib.check(lib.genbmm_logbmm_fwd(p(a), p(b), p(out), p(stats), B, M, K, N, s), "fwd")

    ws = torch.empty(lib.genbmm_logbmm_bwdbwd_ws_size(B, M, K, N), device=dev)

    def bb():  # factored, on the matrix cores
        _lib.check(lib.genbmm_logbmm_bwdbwd_ws(p(a), p(b), p(out), p(g), p(ua), p(ub), p(ga), p(gb), p(gg), p(ws),
                                               B, M, K, N, s), "bwdbwd_ws")

    def bb_ua():  # the reference's case: the cotangent of grad_a only
        _lib.check(lib.genbmm_logbmm_bwdbwd_ws(p(a), p(b), p(out), p(g), p(ua), p(None), p(ga), p(gb), p(gg), p(ws),
                                               B, M, K, N, s), "bwdbwd_ws")

    def bb_exact():  # three vector-ALU passes, one exponential per term in each
        _lib.check(lib.genbmm_logbmm_bwdbwd(p(a), p(b), p(out), p(g), p(ua), p(ub), p(ga), p(gb), p(gg), B, M, K, N, s),
                   "bwdbwd")

    ms = timed(bb, reps)
    bmkn = float(B) * M * K * N
    # three passes over (m, k, n), a weight and a multiply-add or two each: counted as 6 per term
    report("logbmm double backward (%d,%d,%d,%d)" % (B, M, K, N), ms, 6 * bmkn,
           4.0 * B * (3 * M * K + 3 * K * N + 4 * M * N),
           {"ms_u_a_only": round(timed(bb_ua, reps), 4), "ms_exact_passes": round(timed(bb_exact, max(reps // 4, 2)), 4)})


def dense_max(lib, dev, B, M, K, N, reps, prod):
    torch.manual_seed(0)
    if prod:
        a, b = (1 - torch.rand(B, M, K)).to(dev), (1 - torch.rand(B, K, N)).to(dev)
    else:
        a, b = (torch.round(torch.randn(B, M, K) * 8) / 8).to(dev), (torch.round(torch.randn(B, K, N) * 8) / 8).to(dev)
    g = (torch.round(torch.randn(B, M, N) * 8) / 8).clamp(-4, 4).to(dev)
    out = torch.empty(B, M, N, device=dev)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=dev)
    ga, gb = torch.empty_like(a), torch.empty_like(b)
    s, p = _lib.stream_of(a), _lib.ptr
    fac = torch.empty(2, B, M, N, device=dev) if prod else None

    def f():
        if prod:
            _lib.check(lib.genbmm_prodmaxbmm_fwd(p(a), p(b), p(out), p(idx), p(fac), B, M, K, N, s), "fwd")
        else:
            _lib.check(lib.genbmm_maxbmm_fwd(p(a), p(b), p(out), p(idx), B, M, K, N, s), "fwd")

    def bw():
        if prod:
            _lib.check(lib.genbmm_prodmax_bwd(p(a), p(b), p(idx), p(fac), p(g), p(ga), p(gb), B, M, K, N, s), "bwd")
        else:
            _lib.check(lib.genbmm_argmax_bwd(p(idx), p(g), p(ga), p(gb), B, M, K, N, s), "bwd")

    mf, mb = timed(f, reps), timed(bw, reps)
    bmkn = float(B) * M * K * N
    nbytes = 4.0 * B * (2 * M * K + 2 * K * N + 4 * M * N)
    report(("prodmaxbmm" if prod else "maxbmm") + " fwd+bwd (%d,%d,%d,%d)" % (B, M, K, N), mf + mb, 6 * bmkn, nbytes,
           {"ms_fwd": round(mf, 4), "ms_bwd": round(mb, 4)})


def dense_sample(lib, dev, B, M, K, N, reps):
    torch.manual_seed(0)
    a, b = (2 * torch.randn(B, M, K)).to(dev), (2 * torch.randn(B, K, N)).to(dev)
    g = torch.randn(B, M, N).to(dev)
    out = torch.empty(B, M, N, device=dev)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=dev)
    ga, gb = torch.empty_like(a), torch.empty_like(b)
    s, p = _lib.stream_of(a), _lib.ptr

    stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=dev)

    def f():
        _lib.check(lib.genbmm_samplebmm_fwd(p(a), p(b), p(out), p(idx), p(stats), 1234, 0, B, M, K, N, s), "fwd")

    def bw():
        _lib.check(lib.genbmm_argmax_bwd(p(idx), p(g), p(ga), p(gb), B, M, K, N, s), "bwd")

    mf, mb = timed(f, reps), timed(bw, reps)
    bmkn = float(B) * M * K * N
    nbytes = 4.0 * B * (2 * M * K + 2 * K * N + 4 * M * N)
    report("samplebmm fwd+bwd (%d,%d,%d,%d)" % (B, M, K, N), mf + mb, 6 * bmkn, nbytes,
           {"ms_fwd": round(mf, 4), "ms_bwd": round(mb, 4)})


def banded(lib, dev, B, n, lu, ld, mode, reps, pad=None, dtype=torch.float32):
    """pad = (value, rows): the last `rows` band rows of a hold `value`, no gradient flows into them.
    mode 2: the sample product (forward = log product + index walk, backward = one-hot scatter).
    dtype float16 / bfloat16: the `_f16` / `_bf16` entry points on band tensors of that type."""
    torch.manual_seed(7)
    W = lu + ld + 1
    Wo = 2 * W - 1
    a, b = (torch.rand(B, n, W) * 2 - 1).to(dev).to(dtype), (torch.rand(B, n, W) * 2 - 1).to(dev).to(dtype)
    g = torch.randn(B, n, Wo).to(dev).to(dtype)
    if pad is not None:
        a[:, n - pad[1]:, :] = pad[0]
        g[:, n - pad[1]:, :] = 0
    out = torch.empty(B, n, Wo, device=dev, dtype=dtype)
    idx = torch.empty(B, n, Wo, dtype=torch.int32, device=dev) if mode in (1, 2) else None
    ga, gb = torch.empty_like(a), torch.empty_like(b)
    ws = torch.empty(lib.genbmm_banded_workspace_size(lu, ld, lu, ld, B, n), device=dev) if mode in (0, 2) else None
    s, p = _lib.stream_of(a), _lib.ptr
    sfx = _lib.HALF_SUFFIX.get(dtype, "")
    fwd, bwd, smp = (getattr(lib, nm + sfx) for nm in ("genbmm_banded_fwd", "genbmm_banded_bwd", "genbmm_banded_sample_fwd"))

    def f():
        if mode == 2:
            _lib.check(smp(p(a), lu, ld, p(b), lu, ld, p(out), p(idx), p(ws), 1234, 0, B, n, s), "sample fwd")
        else:
            _lib.check(fwd(p(a), lu, ld, p(b), lu, ld, p(out), p(idx), p(ws), B, n, mode, s), "fwd")

    def bw():
        _lib.check(bwd(p(a), lu, ld, p(b), lu, ld, p(out), p(idx), p(None) if mode == 2 else p(ws), p(g), p(ga), p(gb), B, n, mode, s),
                   "bwd")

    mf, mb = timed(f, reps), timed(bw, reps)
    pairs = float(B) * n * W * W
    es = float(a.element_size())
    fb = es * B * n * (2 * W + Wo) + (4.0 * B * n * Wo if mode in (1, 2) else 0)
    bb = es * B * n * (4 * W + Wo) + (es * B * n * Wo if mode == 0 else 0) + (4.0 * B * n * Wo if mode in (1, 2) else 0)
    name = {0: "multiply_log", 1: "multiply_max", 2: "multiply_sample", 3: "multiply"}[mode]
    if sfx:
        name += ", %s bands" % str(dtype).replace("torch.", "")
    report("banded %s fwd+bwd (B=%d,n=%d,lu=ld=%d)%s" % (name, B, n, lu, "" if pad is None else ", last %d rows of a = %g" % (pad[1], pad[0])),
           mf + mb, 6 * pairs, fb + bb,
           {"ms_fwd": round(mf, 4), "ms_bwd": round(mb, 4),
            "fwd_GBs": round(fb / mf / 1e6, 1), "bwd_GBs": round(bb / mb / 1e6, 1)})


def band_structure(lib, dev, B, n, lu, ld, reps):
    """The structural kernels at the banded configuration's size: HBM-bound copies, the
    figure is algorithmic GB/s (one read of the source + one write of the result).  The
    same operation written as torch index arithmetic (the host layer's formulation for
    CPU tensors, run here on the device) is timed beside it."""
    W = lu + ld + 1
    torch.manual_seed(7)
    data = (torch.rand(B, n, W) * 2 - 1).to(dev)
    s, p = _lib.stream_of(data), _lib.ptr
    out = torch.empty_like(data)
    wide = torch.empty(B, n, W + 8, device=dev)
    band_bytes = 4.0 * B * n * W

    def line(name, ms, nbytes, torch_ms=None):
        d = {"config": "band %s (B=%d,n=%d,lu=ld=%d)" % (name, B, n, lu), "ms": round(ms, 4),
             "algorithmic_GBs": round(nbytes / ms / 1e6, 1),
             "pct_hbm_peak": round(100 * nbytes / (ms * 1e-3) / (PEAK_HBM_GBS * 1e9), 2)}
        if torch_ms is not None:
            d["torch_index_ops_ms"] = round(torch_ms, 4)
        print(json.dumps(d), flush=True)

    import torch.nn.functional as F

    def idx_transpose():
        i = torch.arange(n, device=dev).unsqueeze(1)
        k = torch.arange(W, device=dev).unsqueeze(0)
        src = i + k - ld
        ok = (src >= 0) & (src < n)
        g = data[..., src.clamp(0, n - 1), (W - 1 - k).expand_as(src)]
        return torch.where(ok, g, torch.zeros((), device=dev))

    ms = timed(lambda: _lib.check(lib.genbmm_band_transpose(p(data), p(out), B, n, lu, ld, s), "t"), reps)
    line("transpose", ms, 2 * band_bytes, timed(idx_transpose, max(3, reps // 4)))
    ms = timed(lambda: _lib.check(lib.genbmm_band_shift(p(data), p(out), B, n, W, W, 0, 3, 0.0, s), "s"), reps)
    line("band_shift(3)", ms, 2 * band_bytes, timed(lambda: F.pad(data[:, :, 3:], (0, 3)), reps))
    ms = timed(lambda: _lib.check(lib.genbmm_band_shift(p(data), p(out), B, n, W, W, 5, 0, 0.0, s), "c"), reps)
    line("col_shift(5)", ms, 2 * band_bytes, timed(lambda: F.pad(data[:, 5:, :], (0, 0, 0, 5)), reps))
    ms = timed(lambda: _lib.check(lib.genbmm_band_shift(p(data), p(wide), B, n, W, W + 8, 0, -4, 0.0, s), "p"), reps)
    line("band_pad(4)", ms, band_bytes + 4.0 * B * n * (W + 8), timed(lambda: F.pad(data, (4, 4)), reps))
    ms = timed(lambda: _lib.check(lib.genbmm_band_op(p(data), lu, ld, p(data), lu, ld, p(out), B, n, 0, 0.0, s), "o"), reps)
    line("op(add)", ms, 3 * band_bytes, timed(lambda: torch.add(data, data), reps))
    # dense forms: B * n * n * 4 bytes (4.3 GB at B=64, n=4096)
    Bd = B
    dense = torch.empty(Bd, n, n, device=dev)
    sub = data[:Bd].contiguous()
    ms = timed(lambda: _lib.check(lib.genbmm_band_to_dense(p(sub), p(dense), Bd, n, lu, ld, 0.0, s), "d"), reps)
    line("to_dense", ms, 4.0 * Bd * n * (n + W))
    ms = timed(lambda: _lib.check(lib.genbmm_band_from_dense(p(dense), p(out), Bd, n, n, lu, ld, s), "f"), reps)
    line("banddiag", ms, 4.0 * Bd * n * 2 * W)


def dense_f64(lib, dev, B, M, K, N, reps):
    """logbmm / maxbmm forward + backward on the double-precision entry points (plain
    kernels: the figure of merit is % of the FP64 vector peak, 78.6 TFLOP/s)."""
    torch.manual_seed(0)
    a, b, g = (torch.randn(B, M, K).double().to(dev), torch.randn(B, K, N).double().to(dev),
               torch.randn(B, M, N).double().to(dev))
    out = torch.empty(B, M, N, dtype=torch.float64, device=dev)
    idx = torch.empty(B, M, N, dtype=torch.int32, device=dev)
    ga, gb = torch.empty_like(a), torch.empty_like(b)
    s, p = _lib.stream_of(a), _lib.ptr
    bmkn = float(B) * M * K * N
    for name, f, bw in (
        ("logbmm", lambda: lib.genbmm_logbmm_fwd_f64(p(a), p(b), p(out), B, M, K, N, s),
         lambda: lib.genbmm_logbmm_bwd_f64(p(a), p(b), p(out), p(g), p(ga), p(gb), B, M, K, N, s)),
        ("maxbmm", lambda: lib.genbmm_maxbmm_fwd_f64(p(a), p(b), p(out), p(idx), B, M, K, N, s),
         lambda: lib.genbmm_argmax_bwd_f64(p(idx), p(g), p(ga), p(gb), B, M, K, N, s)),
    ):
        mf = timed(lambda: _lib.check(f(), "fwd"), reps)
        mb = timed(lambda: _lib.check(bw(), "bwd"), reps)
        ms = mf + mb
        print(json.dumps({"config": "%s f64 fwd+bwd (%d,%d,%d,%d)" % (name, B, M, K, N), "ms": round(ms, 4),
                          "semiring_GOPs": round(6 * bmkn / ms / 1e6, 1),
                          "pct_fp64_vector_peak": round(100 * 6 * bmkn / (ms * 1e-3) / 78.6e12, 2),
                          "ms_fwd": round(mf, 4), "ms_bwd": round(mb, 4)}), flush=True)


def cpu_c1():
    import oracle

    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    torch.manual_seed(0)
    a = torch.rand(16, 64, 64, requires_grad=True)
    b = torch.rand(16, 64, 64, requires_grad=True)

    def one():
        a.grad = b.grad = None
        oracle.logbmm_broadcast(a, b).backward(torch.ones(16, 64, 64))

    one()
    ts = []
    for _ in range(11):
        t0 = time.perf_counter()
        one()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    ops = 6.0 * 16 * 64 * 64 * 64
    print(json.dumps({"config": "logbmm fwd+bwd (16,64,64,64) CPU torch broadcast", "ms": round(ts[5] * 1e3, 3),
                      "semiring_GOPs": round(ops / ts[5] / 1e9, 2), "cores": torch.get_num_threads()}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--cpu", action="store_true")
    ap.add_argument("--only", default="", help="comma-separated subset: log,half,max,sample,banded,struct,f64; "
                    "widths (not in the default set): the banded products at 5 ... 81 diagonals per operand; "
                    "pad (not in the default set): the log products with whole rows of padding (-1e9, -1e5, -inf)")
    args = ap.parse_args()
    want = set(args.only.split(",")) if args.only else {"log", "half", "max", "sample", "banded", "struct", "f64"}
    lib = _lib.load()
    dev = torch.device("cuda:0")
    r = args.reps
    if "log" in want:
        dense_log(lib, dev, 16, 64, 64, 64, r, "logbmm fwd+bwd (16,64,64,64) config 0", dist="rand", graph=True)
        dense_log(lib, dev, 512, 128, 128, 128, r, "logbmm fwd+bwd (512,128,128,128) config 1")
        dense_log(lib, dev, 8192, 32, 32, 32, r, "logbmm fwd+bwd (8192,32,32,32) config 1 skinny")
        dense_log2(lib, dev, 512, 128, 128, 128, max(3, r // 4))
        for path in (0, 4, 3, 2, 1):
            dense_log(lib, dev, 64, 512, 512, 512, r, "logbmm fwd+bwd (64,512,512,512) headline", path=path)
    if "half" in want:
        for dt, nm in ((torch.float16, "float16"), (torch.bfloat16, "bfloat16")):
            dense_log(lib, dev, 64, 512, 512, 512, r, "logbmm fwd+bwd (64,512,512,512) headline, %s tensors" % nm, dtype=dt)
            dense_log(lib, dev, 512, 128, 128, 128, r, "logbmm fwd+bwd (512,128,128,128) config 1, %s tensors" % nm, dtype=dt)
            dense_log(lib, dev, 8192, 32, 32, 32, r, "logbmm fwd+bwd (8192,32,32,32) config 1 skinny, %s tensors" % nm, dtype=dt)
    if "max" in want:
        dense_max(lib, dev, 256, 256, 256, 256, r, prod=False)
        dense_max(lib, dev, 256, 256, 256, 256, r, prod=True)
    if "sample" in want:
        dense_sample(lib, dev, 64, 512, 512, 512, r)
        dense_sample(lib, dev, 16, 512, 1024, 512, r)  # K beyond the 62 slabs of the sweep's six-bit tag
    if "banded" in want:
        for mode in (3, 0, 1, 2):
            banded(lib, dev, 64, 4096, 32, 32, mode, r)
        for dt in (torch.float16, torch.bfloat16):
            for mode in (3, 0, 1):
                banded(lib, dev, 64, 4096, 32, 32, mode, r, dtype=dt)
    if "widths" in want:
        for lu in (2, 4, 8, 16, 24, 32, 40):
            for mode in (3, 0, 1):
                banded(lib, dev, 64, 4096, lu, lu, mode, r)
    if "pad" in want:
        for value in (-1e9, -1e5, float("-inf")):
            for (B, M, K, N, rows) in ((64, 512, 512, 512, 8), (512, 128, 128, 128, 4), (2048, 64, 64, 64, 4), (8192, 32, 32, 32, 4)):
                dense_log(lib, dev, B, M, K, N, r, "logbmm fwd+bwd (%d,%d,%d,%d), last %d rows of a = %g" % (B, M, K, N, rows, value),
                          pad=(value, rows))
            if value != float("-inf"):
                banded(lib, dev, 64, 4096, 32, 32, 0, r, pad=(value, 400))
    if "struct" in want:
        band_structure(lib, dev, 64, 4096, 32, 32, r)
    if "f64" in want:
        dense_f64(lib, dev, 512, 128, 128, 128, max(3, r // 4))
    if args.cpu:
        cpu_c1()


if __name__ == "__main__":
    main()

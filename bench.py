"""Benchmark of the GCN hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--scale S] [--no-cpu] [--spmm-only]

Workload (default): the 3-layer GCN configuration on a synthetic power-law graph with 2,449,029 nodes
and about 126 M stored entries (Chung-Lu, exponent 2.1, self loops, GCN normalisation, random vertex
permutation); features 2,449,029 x 100, hidden 128, 47 classes, fp32.  A step is one training epoch:
zero_grad, forward (3 x [SpMM, GEMM(+ReLU)]), fused cross-entropy, backward (3 x [GEMM^T, GEMM, SpMM]),
AdamW over weights and features.  All inputs are resident in HBM before the timed region.

The JSON line's ``value`` is the SpMM's algorithmic bandwidth: the bytes every operand of
AGG = A.H (D = 128) must move once, divided by the measured time of the product.  ``roofline`` describes
its dominant kernel (the row kernel; on this graph the longest rows are taken by a second kernel, the hub pass, and
``spmm_parts`` gives both); ``cpu_baseline`` is the same product computed by the reference's operator
(torch.sparse.mm on the host cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
FP32_VECTOR_TFLOPS = 157.3
# Bytes moved between L2 and the memory side per SpMM launch, from rocprofv3 counters (FETCH_SIZE and WRITE_SIZE, each
# scaled by what the same counter reads for a plain 1 GiB copy).  The figures are not kept here: they are read from the
# trailer of the counter summary under profiles/, which also names the commit it was taken at, and both are reported
# in the JSON line (roofline.traffic, roofline.traffic_source).
SPMM_TRAFFIC_PROFILE = os.path.join("profiles", "spmm_csr_config3_fp32_pmc.txt")


def measured_spmm_traffic(n, nnz, d):
    """(bytes per launch or None, where the figure comes from) for the SpMM of an n-row, nnz-entry graph at width d."""
    import re

    path = os.path.join(ROOT, SPMM_TRAFFIC_PROFILE)
    try:
        text = open(path).read()
    except OSError:
        return None, None
    commit = re.search(r"^\s*taken_at_commit\s*=\s*(\S+)", text, flags=re.M)
    kernel = re.search(r"^\s*kernel\s*=\s*(.+)$", text, flags=re.M)
    m = re.search(r"^\s*traffic_bytes_per_launch\[%d,%d,%d\]\s*=\s*([0-9.eE+]+)" % (n, nnz, d), text, flags=re.M)
    if not m:
        return None, None
    source = {"profile": SPMM_TRAFFIC_PROFILE, "commit": commit.group(1) if commit else None,
              "kernel": kernel.group(1).strip() if kernel else None}
    hub = re.search(r"^\s*hub_traffic_bytes_per_launch\[%d,%d,%d\]\s*=\s*([0-9.eE+]+)" % (n, nnz, d), text, flags=re.M)
    source["hub_pass_traffic"] = float(hub.group(1)) if hub else None
    return float(m.group(1)), source


def spmm_bytes(m, k, nnz, d, elem=4):
    """int32 column + fp32 value per entry, int32 row pointers, H read once, Y written once."""
    return nnz * (4 + 4) + (m + 1) * 4 + k * d * elem + m * d * elem


def time_gpu(fn, warmup, iters):
    import torch

    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def bench_side_config(args, dev):
    """Configurations 2 and 4 (parity-test cases; timed here so that the figures quoted for them can be re-measured).

    Config 2: SpMM only on the R-MAT graph (232,965 nodes, about 114.6 M entries), H 232,965 x 602 and x 128;
    a step is one SpMM at D = 602.  Config 4: one rank's block of a 2 x 2 x 2 grid (rows and columns [0, N/2) of a
    doubly permuted R-MAT graph with N = 8,388,608), local widths 64 -> 64 -> 64 -> 24; a step is forward, loss and
    backward of the three layers on that block (no optimizer: the rank's share of an epoch without collectives)."""
    import torch

    from plexus_amd import ops
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.train import Net
    from plexus_amd.utils import synthetic as S

    t0 = time.time()
    g = S.config2_graph(dev, seed=0, scale=args.scale) if args.config == 2 else S.config4_block(dev, seed=0, scale=args.scale)
    m, k = g.shape
    nnz = g.nnz
    stats = g.degree_stats()
    a = ops.CsrMatrix(g.rowptr, g.col, g.val, g.shape, args.seg_len)
    torch.cuda.synchronize()
    print("# graph: %s, long rows %d, segments %d, generated and prepared in %.1f s" % (stats, a.n_long_rows, a.n_segments, time.time() - t0),
          file=sys.stderr, flush=True)
    widths = (602, 128) if args.config == 2 else (64,)
    spmm = {}
    for d in widths:
        h = S.normal_features(k, d, dev, seed=d)
        out = torch.empty(m, d, device=dev)
        ms = time_gpu(lambda: ops.spmm(a, h, out=out), 5, args.spmm_iters)
        b = spmm_bytes(m, k, nnz, d)
        spmm[d] = {"ms": ms, "alg_bytes": b, "alg_GBps": b / ms / 1e6, "GFLOPs": 2.0 * nnz * d / ms / 1e6,
                   "gather_GBps": (nnz * 8 + (m + 1) * 4 + nnz * d * 4 + m * d * 4) / ms / 1e6}
        print("# spmm D=%d fp32: %.3f ms, %.1f GB/s algorithmic, %.1f GFLOP/s, gather model %.0f GB/s"
              % (d, ms, spmm[d]["alg_GBps"], spmm[d]["GFLOPs"], spmm[d]["gather_GBps"]), file=sys.stderr, flush=True)
        if d == widths[0]:
            h0, out0 = h, out  # kept for the comparison with the host operator
        del h, out
    dom = spmm[widths[0]]
    step_ms = dom["ms"]
    extra = {}
    if args.config == 4 and not args.spmm_only:
        at = ops.csr_transpose(a, args.seg_len)
        dims = [64, 64, 64, 24]
        x = S.normal_features(k, dims[0], dev, seed=1).reshape(-1).requires_grad_()
        y = S.uniform_labels(m, dims[-1], dev, seed=2)
        model = Net(3, dims[0], dims[1], dims[-1], weights=S.glorot_weights(dims, seed=0), fuse_relu=True)

        def one_step():
            x.grad = None
            for layer in model.layers:
                layer.weight.grad = None
            loss = parallel_cross_entropy(model(x, [(a, at)]), y, 3, m, dims[-1])
            loss.backward()
            return loss

        step_ms = time_gpu(one_step, args.warmup, args.steps)
        extra["block_fwd_bwd_ms"] = step_ms
        print("# block forward + loss + backward (64-64-64-24): %.2f ms" % step_ms, file=sys.stderr, flush=True)
    cpu = None
    if not args.no_cpu:
        from oracle import plexus_oracle as po

        a_cpu = torch.sparse_csr_tensor(g.rowptr.cpu(), g.col.cpu(), g.val.cpu(), size=g.shape)
        h_cpu = h0.cpu()
        po.spmm(a_cpu, h_cpu)
        t2 = time.time()
        y_cpu = po.spmm(a_cpu, h_cpu)
        cpu_s = time.time() - t2
        err = ((ops.spmm(a, h0).cpu().double() - y_cpu.double()).abs().max() / y_cpu.double().abs().max()).item()
        cpu = {"value": dom["alg_bytes"] / cpu_s / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
               "sample": "the whole SpMM of the workload at D=%d (torch.sparse.mm, fp32, 1 timed run after 1 warm-up)" % widths[0],
               "ms": cpu_s * 1e3, "GFLOPs": 2.0 * nnz * widths[0] / cpu_s / 1e9, "max_rel_err_gpu_vs_cpu": err}
        print("# cpu: %.0f ms per SpMM on %d threads, gpu-vs-cpu max rel err %.2e" % (cpu_s * 1e3, cpu["cores"], err), file=sys.stderr, flush=True)
    what = ("config 2: SpMM only, R-MAT graph, N=%d, nnz=%d (value and step = A.H at D=602)" % (m, nnz) if args.config == 2 else
            "config 4: one rank's %d x %d block of a 2x2x2 grid, nnz=%d (value = A.H at D=64; step = 3-layer forward + loss + "
            "backward on the block, widths 64-64-64-24, no collectives)" % (m, k, nnz))
    line = {"metric": "SpMM HBM GB/s (% of peak) + GCN fwd+bwd epoch ms on 1 MI355X", "value": dom["alg_GBps"], "unit": "GB/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": step_ms, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": what, "rows": m, "cols": k, "nnz": nnz, "max_row_nnz": stats["max_row_nnz"], "scale": args.scale,
                       "split_rows": a.n_long_rows, "segments": a.n_segments},
            "spmm": {str(d): v for d, v in spmm.items()},
            "roofline": {"bound": "hbm", "achieved": dom["alg_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": dom["alg_GBps"] / HBM_PEAK_GBPS, "traffic": None,
                         "kernel": "spmm_csr_kernel (A.H, D=%d, fp32)" % widths[0], "alg_bytes_per_launch": dom["alg_bytes"],
                         "avg_launch_ms": dom["ms"]},
            "cpu_baseline": cpu}
    line.update(extra)
    print(json.dumps(line), flush=True)


def bench_config1(args, dev):
    """Configuration 1, the reference's own CPU-runnable case (2,708 nodes, 1433 -> 16 -> 7, ten AdamW epochs): a
    parity-test case, timed here beside the oracle harness on the host.  A step is one epoch; the work is bound by
    launch latency, so forward + loss + backward is also timed as one HIP-graph replay."""
    import torch

    from oracle import plexus_oracle as po
    from plexus_amd.cross_entropy import parallel_cross_entropy
    from plexus_amd.train import Net, make_optimizer, run_epochs
    from plexus_amd.utils import synthetic as S

    g, x, y, dims = S.config1(device="cpu", seed=0)
    n = g.shape[0]
    weights = S.glorot_weights(dims, seed=0)
    shards = [(g.torch_csr().to(dev), g.torch_csr(True).to(dev))]
    yd = y.to(dev)

    def gpu_run():
        model = Net(2, dims[0], dims[1], dims[2], weights=weights, fuse_relu=True)
        feats = x.reshape(-1).to(dev).requires_grad_()
        opt = make_optimizer(model, feats)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        losses = run_epochs(model, opt, feats, shards, yd, n, dims[-1], 10)
        torch.cuda.synchronize()
        return losses, (time.perf_counter() - t0) * 1e3

    gpu_run()  # warm-up: library load, plans, allocator
    losses, gpu_ms = min((gpu_run() for _ in range(max(args.steps // 10, 3))), key=lambda r: r[1])

    # forward + loss + backward as one graph replay
    model = Net(2, dims[0], dims[1], dims[2], weights=weights, fuse_relu=True)
    feats = x.reshape(-1).to(dev).requires_grad_()
    params = list(model.parameters()) + [feats]

    def fwd_bwd():
        for p in params:
            p.grad = None
        loss = parallel_cross_entropy(model(feats, shards), yd, 2, n, dims[-1])
        loss.backward()
        return loss

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fwd_bwd()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fwd_bwd()
    eager_ms = time_gpu(fwd_bwd, 10, 200)
    replay_ms = time_gpu(graph.replay, 10, 200)

    cpu = None
    if not args.no_cpu:
        adj = [(g.torch_csr(), g.torch_csr(True))]
        po.train_epochs(x, weights, dims, adj, y, n, dims[-1], epochs=1)
        t0 = time.perf_counter()
        ref_losses, _, _ = po.train_epochs(x, weights, dims, adj, y, n, dims[-1], epochs=10)
        cpu_ms = (time.perf_counter() - t0) * 1e3
        worst = max(abs(a - b) / abs(b) for a, b in zip(losses, ref_losses))
        cpu = {"value": cpu_ms / 10, "unit": "ms per epoch", "cores": torch.get_num_threads(), "kind": "port",
               "sample": "the whole workload: ten epochs of the oracle harness (torch CPU operators, fp32)",
               "max_rel_loss_difference_gpu_vs_cpu": worst}
    line = {"metric": "GCN fwd+bwd epoch ms on 1 MI355X (config 1)", "value": gpu_ms / 10, "unit": "ms", "n_gpus": 1, "steps": 10,
            "warmup": 10, "ms_per_step": gpu_ms / 10, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32", "data": "synthetic",
            "config": {"workload": "config 1: 2-layer GCN 1433-16-7, N=%d, nnz=%d, ten AdamW epochs over weights and features"
                                   % (n, g.nnz)},
            "losses": losses, "fwd_loss_bwd_eager_ms": eager_ms, "fwd_loss_bwd_graph_replay_ms": replay_ms,
            "roofline": None, "cpu_baseline": cpu}
    print(json.dumps(line), flush=True)


def bench_dense_kernels(args, dev):
    """The dense products, the loss and the optimizer of config 3 (or 5) one by one, at the workload's shapes, with
    their algorithmic bytes and flops: the kernels that a counter run of this mode profiles."""
    import torch

    from plexus_amd import ops
    from plexus_amd.optim import AdamW
    from plexus_amd.utils import synthetic as S

    m = max(64, int(2449029 * args.scale))
    bf16 = args.config == 5
    dims = [256, 256, 256, 47] if bf16 else [100, 128, 128, 47]
    e = 2 if bf16 else 4
    rows = []

    def rec(name, fn, bytes_, flops):
        ms = time_gpu(fn, 3, args.spmm_iters)
        rows.append({"kernel": name, "ms": ms, "GBps": bytes_ / ms / 1e6, "TFLOPs": flops / ms / 1e9,
                     "frac_hbm_peak": bytes_ / ms / 1e6 / HBM_PEAK_GBPS})
        print("# %-44s %7.3f ms  %7.0f GB/s (%4.1f %% of HBM peak)  %6.1f TFLOP/s" % (name, ms, rows[-1]["GBps"], 100 * rows[-1]["frac_hbm_peak"],
                                                                                 rows[-1]["TFLOPs"]), file=sys.stderr, flush=True)

    for li in range(3):
        k, n = dims[li], dims[li + 1]
        last = li == 2
        if bf16:
            a = S.normal_features(m, k, dev, seed=li, dtype=torch.bfloat16)
            g = S.normal_features(m, n, dev, seed=10 + li, dtype=torch.bfloat16)
            w = torch.randn(k, n, device=dev) * 0.1
            wt16, w16 = ops.cast_bf16(w, transpose=True), ops.cast_bf16(w)
            act = torch.relu(S.normal_features(m, n, dev, seed=20 + li)).to(torch.bfloat16)
            rec("OUT = AGG.W %dx%d bf16%s" % (k, n, "" if last else " +ReLU +dropout"),
                (lambda: ops.gemm_nt_bf16(a, wt16)) if last else (lambda: ops.gemm_nt_bf16(a, wt16, relu=True, dropout_p=0.5, seed=1, offset=li)),
                e * m * (k + n), 2.0 * m * k * n)
            rec("GRAD_AGG = (G*mask).W^T %dx%d bf16" % (n, k), (lambda: ops.gemm_nt_bf16(g, w16)) if last else (lambda: ops.gemm_nt_bf16(g, w16, mask=act, alpha=2.0)),
                e * m * (k + n) + (0 if last else e * m * n), 2.0 * m * k * n)
            rec("GRAD_W = AGG^T.(G*mask) %dx%d bf16" % (k, n), (lambda: ops.gemm_tn_bf16(a, g)) if last else (lambda: ops.gemm_tn_bf16(a, g, mask=act, alpha=2.0)),
                e * m * (k + n) + (0 if last else e * m * n), 2.0 * m * k * n)
        else:
            a = S.normal_features(m, k, dev, seed=li)
            g = S.normal_features(m, n, dev, seed=10 + li)
            w = torch.randn(k, n, device=dev) * 0.1
            wt = w.t().contiguous()
            act = torch.relu(S.normal_features(m, n, dev, seed=20 + li))
            # a hidden layer's product also writes the sign bits of its result, and GRAD_AGG reads the mask in that form
            bits = None if last else ops.sign_bits(act)
            rec("OUT = AGG.W %dx%d%s" % (k, n, "" if last else " +ReLU +sign bits"),
                (lambda: ops.gemm_nn(a, w)) if last else (lambda: ops.gemm_nn(a, w, relu=True, want_bits=True)),
                e * m * (k + n) + (0 if last else m * n // 8), 2.0 * m * k * n)
            rec("GRAD_AGG = (G*mask).W^T %dx%d%s" % (n, k, "" if last else " (bit mask)"),
                (lambda: ops.gemm_nt(g, w)) if last else (lambda: ops.gemm_nt(g, w, mask=act, mask_bits=bits)),
                e * m * (k + n) + (0 if last else m * n // 8), 2.0 * m * k * n)
            rec("GRAD_W = AGG^T.(G*mask) %dx%d" % (k, n), lambda: ops.gemm_tn(a, g, mask=None if last else act),
                e * m * (k + n) + (0 if last else e * m * n), 2.0 * m * k * n)
            del wt
        del a, g, act
    logits = S.normal_features(m, dims[-1], dev, seed=3, dtype=torch.bfloat16 if bf16 else torch.float32)
    labels = S.uniform_labels(m, dims[-1], dev, seed=2)
    rec("cross-entropy loss + gradient, %d classes" % dims[-1], lambda: ops.softmax_xent(logits, labels, m, dims[-1]), 2 * e * m * dims[-1] + 8 * m, 0.0)
    del logits
    n_feat = m * dims[0]
    p = torch.randn(n_feat, device=dev).requires_grad_()
    if bf16:
        shadow = p.detach().to(torch.bfloat16).requires_grad_()
        shadow.grad = torch.randn(n_feat, device=dev).to(torch.bfloat16)
        opt = AdamW([p], lr=3e-3, weight_decay=0.0, shadows=[(p, shadow)])
        rec("AdamW over the features (fp32 master, bf16 gradient and copy)", opt.step, 30 * n_feat, 0.0)
    else:
        p.grad = torch.randn(n_feat, device=dev)
        opt = AdamW([p], lr=3e-3, weight_decay=0.0)
        rec("AdamW over the features", opt.step, 28 * n_feat, 0.0)
    line = {"metric": "dense products, loss and optimizer of the workload, one by one", "value": sum(r["ms"] for r in rows), "unit": "ms",
            "n_gpus": 1, "steps": args.spmm_iters, "warmup": 3, "ms_per_step": sum(r["ms"] for r in rows), "higher_is_better": False,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if bf16 else "f32", "data": "synthetic",
            "config": {"workload": "config %d dense kernels at M=%d, widths %s" % (args.config, m, "-".join(map(str, dims)))},
            "kernels": rows}
    print(json.dumps(line), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the graph (for quick checks)")
    ap.add_argument("--seg-len", type=int, default=0, help="split rows longer than this (0 = library default)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host baseline")
    ap.add_argument("--no-cpu-epoch", action="store_true", help="host baseline: time the SpMM only, not a whole epoch")
    ap.add_argument("--spmm-only", action="store_true", help="time only the SpMM kernels")
    ap.add_argument("--dense-only", action="store_true",
                    help="time the dense products, the loss and the optimizer of the workload one by one (no graph)")
    ap.add_argument("--spmm-iters", type=int, default=20)
    ap.add_argument("--config", type=int, default=3, choices=[1, 2, 3, 4, 5],
                    help="3: fp32, 100-128-128-47 (default, the headline workload); 5: bf16 storage, 256-256-256-47, dropout 0.5; "
                         "2: SpMM only on the R-MAT graph; 4: one rank's block of a 2x2x2 grid; "
                         "1: the 2,708-node CPU-runnable case, ten epochs")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch a plain 1 GiB device copy (known size) to calibrate profiler byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives are implemented); --gpus %d is not "
              "supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch

    from plexus_amd import _lib, ops
    from plexus_amd.train import Net, make_optimizer, train
    from plexus_amd.utils import synthetic as S

    _lib.load()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(2)
    dev = "cuda"
    torch.cuda.set_device(0)
    if args.config == 1:
        return bench_config1(args, dev)
    if args.config in (2, 4):
        return bench_side_config(args, dev)
    if args.dense_only:
        return bench_dense_kernels(args, dev)

    t0 = time.time()
    g = S.config3_graph(dev, seed=0, scale=args.scale)
    n = g.shape[0]
    stats = g.degree_stats()
    torch.cuda.synchronize()
    gen_s = time.time() - t0
    # preparation, timed apart from the hot path: int64 -> int32 indices + row plan, and the device-side transpose.
    # Each is run twice and the second run is reported: the first call into the library also loads its code object
    # and makes the allocator fetch fresh memory (about 25 ms each, once per process; kept as *_first_call).
    def timed_twice(fn):
        out, ms = None, []
        for _ in range(2):
            del out
            torch.cuda.synchronize()
            t_prep = time.time()
            out = fn()
            torch.cuda.synchronize()
            ms.append((time.time() - t_prep) * 1e3)
        return out, ms[1], ms[0]

    a, prep_plan_ms, prep_plan_first_ms = timed_twice(lambda: ops.CsrMatrix(g.rowptr, g.col, g.val, g.shape, args.seg_len))
    at, prep_transpose_ms, prep_transpose_first_ms = timed_twice(lambda: ops.csr_transpose(a, args.seg_len))
    assert torch.equal(at.col, g.col_t.to(torch.int32)) and torch.equal(at.val, g.val_t)  # same as the generator's own transpose
    nnz = g.nnz
    bf16 = args.config == 5
    dims = [256, 256, 256, 47] if bf16 else [100, 128, 128, 47]
    dtype = torch.bfloat16 if bf16 else torch.float32
    elem = 2 if bf16 else 4
    d_main, d_side = (256, 128) if bf16 else (128, 100)
    print("# graph: %s, long rows %d, segments %d, generated in %.1f s; narrow+plan %.1f ms, device transpose+plan %.1f ms"
          % (stats, a.n_long_rows, a.n_segments, gen_s, prep_plan_ms, prep_transpose_ms), file=sys.stderr, flush=True)

    if args.calib_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # ---- the dominant kernel: SpMM at D = 128 (and D = 100 beside it) ----
    spmm = {}
    for d in (d_main, d_side):
        h = S.normal_features(n, d, dev, seed=d, dtype=dtype)
        out = torch.empty(n, d, device=dev, dtype=dtype)
        ms = time_gpu(lambda: ops.spmm(a, h, out=out), 5, args.spmm_iters)
        b = spmm_bytes(n, n, nnz, d, elem)
        flops = 2.0 * nnz * d
        spmm[d] = {"ms": ms, "alg_bytes": b, "alg_GBps": b / ms / 1e6, "GFLOPs": flops / ms / 1e6,
                   "gather_GBps": (nnz * 8 + (n + 1) * 4 + nnz * d * elem + n * d * elem) / ms / 1e6,
                   "t_roof_ms": max(b / (HBM_PEAK_GBPS * 1e6), flops / (FP32_VECTOR_TFLOPS * 1e9))}
        print("# spmm D=%d %s: %.3f ms, %.1f GB/s algorithmic, %.1f GFLOP/s" % (d, "bf16" if bf16 else "fp32", ms, spmm[d]["alg_GBps"], spmm[d]["GFLOPs"]),
              file=sys.stderr, flush=True)
        del h, out
    dom = spmm[d_main]

    # ceiling of the memory system for this access pattern: random rows of a table as large as H, nothing else
    gather_ceiling = None
    if not bf16:
        import ctypes

        tab = S.normal_features(n, 128, dev, seed=3)
        sink = torch.zeros(1, device=dev)
        done = ctypes.c_int64(0)
        lib = _lib.load()
        call = lambda: _lib.check(lib.plx_diag_random_gather_f32(tab.data_ptr(), n, 128, 128, nnz, ctypes.byref(done), sink.data_ptr(),
                                                                 torch.cuda.current_stream().cuda_stream), "plx_diag_random_gather_f32")
        ms = time_gpu(call, 2, 5)
        gather_ceiling = {"GBps": done.value * 512 / ms / 1e6, "table_MB": n * 512 / 1e6, "row_bytes": 512,
                          "spmm_gather_GBps": nnz * 512 / dom["ms"] / 1e6}
        print("# random 512-byte row gathers on a %.0f MB table: %.0f GB/s; the SpMM gathers %.0f GB/s of rows of H"
              % (gather_ceiling["table_MB"], gather_ceiling["GBps"], gather_ceiling["spmm_gather_GBps"]), file=sys.stderr, flush=True)
        del tab

    # ---- the two parts of a product with a hub pass, each timed by itself ----
    # The row kernel (spmm_csr_kernel) takes the rows that are not hub rows, one wavefront per row or segment; the hub
    # pass (spmm_hub_kernel) takes the longest rows.  Algorithmic bytes of a part: its entries (int32 column + fp32
    # value, and for the hub pass the 5 bytes per entry of its streams), the row pointers, H once, its rows of Y once.
    parts = None
    if not bf16 and a.n_hub_rows > 0:
        from plexus_amd import _lib

        lib = _lib.load()
        h = S.normal_features(n, d_main, dev, seed=d_main)
        out = torch.empty(n, d_main, device=dev)
        ws, ws_bytes = a._workspace(d_main)

        def run_part(which):
            _lib.check(lib.plx_diag_spmm_parts_f32(a._plan, a.val.data_ptr(), h.data_ptr(), d_main, d_main, out.data_ptr(), d_main,
                                                   ws.data_ptr() if ws is not None else None, ws_bytes, which,
                                                   torch.cuda.current_stream().cuda_stream), "plx_diag_spmm_parts_f32")

        hub_nnz, hub_rows = a.hub_entries, a.n_hub_rows
        rows_ms = time_gpu(lambda: run_part(1), 3, args.spmm_iters)
        hub_ms = time_gpu(lambda: run_part(2), 3, args.spmm_iters)
        rows_bytes = (nnz - hub_nnz) * 8 + (n + 1) * 4 + n * d_main * 4 + (n - hub_rows) * d_main * 4
        hub_bytes = hub_nnz * (8 + 5) + n * d_main * 4 + hub_rows * d_main * 4
        parts = {"row_kernel": {"kernel": "spmm_csr_kernel", "ms": rows_ms, "entries": nnz - hub_nnz, "rows": n - hub_rows,
                                "alg_bytes": rows_bytes, "alg_GBps": rows_bytes / rows_ms / 1e6},
                 "hub_pass": {"kernel": "spmm_hub_kernel", "ms": hub_ms, "entries": hub_nnz, "rows": hub_rows,
                              "alg_bytes": hub_bytes, "alg_GBps": hub_bytes / hub_ms / 1e6}}
        src = measured_spmm_traffic(n, nnz, d_main)[1]
        parts["hub_pass"]["traffic"] = src["hub_pass_traffic"] if src else None
        print("# spmm D=%d in parts: row kernel %.3f ms (%.1f %% of the entries), hub pass %.3f ms (%d rows, %.1f %% of the entries)"
              % (d_main, rows_ms, 100.0 * (nnz - hub_nnz) / nnz, hub_ms, hub_rows, 100.0 * hub_nnz / nnz), file=sys.stderr, flush=True)
        del h, out

    # ---- the epoch ----
    epoch_ms = None
    epoch_ms_tf = None
    losses = []
    if not args.spmm_only:
        y = S.uniform_labels(n, dims[-1], dev, seed=2)
        if bf16:
            # fp32 master features for the optimizer, bf16 copy read by the model and refreshed by the update
            x_master = S.normal_features(n, dims[0], dev, seed=1).reshape(-1)
            x = x_master.to(torch.bfloat16).requires_grad_()
            model = Net(3, dims[0], dims[1], dims[-1], weights=S.glorot_weights(dims, seed=0), fuse_relu=True, dropout=0.5,
                        dropout_seed=0)
            opt = make_optimizer(model, x_master, features_bf16=x)
        else:
            x = S.normal_features(n, dims[0], dev, seed=1).reshape(-1).requires_grad_()
            model = Net(3, dims[0], dims[1], dims[-1], weights=S.glorot_weights(dims, seed=0), fuse_relu=True)
            opt = make_optimizer(model, x)
        shards = [(a, at)]
        for _ in range(args.warmup):
            losses.append(float(train(model, opt, x, shards, y, n, dims[-1])))
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t1 = time.time()
        start.record()
        for _ in range(args.steps):
            loss = train(model, opt, x, shards, y, n, dims[-1])
        stop.record()
        torch.cuda.synchronize()
        wall_ms = (time.time() - t1) * 1e3 / args.steps
        epoch_ms = start.elapsed_time(stop) / args.steps
        losses.append(float(loss))
        print("# epoch: %.2f ms (wall %.2f ms), loss %.4f -> %.4f" % (epoch_ms, wall_ms, losses[0], losses[-1]),
              file=sys.stderr, flush=True)
        if True:
            # the same epoch with the narrowing last layer computed as A.(H.W) (an option of this build; the
            # reference always aggregates first, and the headline number above keeps the reference's order)
            del model, opt
            if bf16:
                x2_master = S.normal_features(n, dims[0], dev, seed=1).reshape(-1)
                x2 = x2_master.to(torch.bfloat16).requires_grad_()
                model2 = Net(3, dims[0], dims[1], dims[-1], weights=S.glorot_weights(dims, seed=0), fuse_relu=True, dropout=0.5,
                             dropout_seed=0, association="auto")
                opt2 = make_optimizer(model2, x2_master, features_bf16=x2)
            else:
                x2 = S.normal_features(n, dims[0], dev, seed=1).reshape(-1).requires_grad_()
                model2 = Net(3, dims[0], dims[1], dims[-1], weights=S.glorot_weights(dims, seed=0), fuse_relu=True, association="auto")
                opt2 = make_optimizer(model2, x2)
            for _ in range(args.warmup):
                train(model2, opt2, x2, shards, y, n, dims[-1])
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(args.steps):
                loss2 = train(model2, opt2, x2, shards, y, n, dims[-1])
            e1.record()
            torch.cuda.synchronize()
            epoch_ms_tf = e0.elapsed_time(e1) / args.steps
            print("# epoch with transform-first last layer: %.2f ms, loss -> %.4f" % (epoch_ms_tf, float(loss2)), file=sys.stderr, flush=True)
            del model2, opt2, x2

    # ---- preprocessing on the device, timed apart: GCN normalisation and the double permutation ----
    prep_norm_ms = prep_perm_ms = None
    if not args.spmm_only:
        from plexus_amd.utils import dataset as D

        raw_ei, _ = ops.csr_to_edges(a)  # the graph's edges (self loops included), unit weights
        torch.cuda.synchronize()
        t_prep = time.time()
        a_hat = D.gcn_norm(raw_ei, None, n)
        torch.cuda.synchronize()
        prep_norm_ms = (time.time() - t_prep) * 1e3
        assert torch.equal(a_hat.col, a.col) and float((a_hat.val - a.val).abs().max()) <= 1e-6  # the generator's own normalisation
        host_gen = torch.Generator().manual_seed(0)
        p1, p2 = torch.randperm(n, generator=host_gen).to(dev), torch.randperm(n, generator=host_gen).to(dev)
        torch.cuda.synchronize()
        t_prep = time.time()
        e1, w1 = D.permute_adjacency(a_hat, p1, p2)
        e2, w2 = D.permute_adjacency(a_hat, p2, p1)
        torch.cuda.synchronize()
        prep_perm_ms = (time.time() - t_prep) * 1e3
        print("# preprocessing on the device: GCN norm from the edge list %.1f ms, double permutation (two adjacencies) %.1f ms"
              % (prep_norm_ms, prep_perm_ms), file=sys.stderr, flush=True)
        del raw_ei, a_hat, e1, w1, e2, w2, p1, p2

    # ---- host baseline: the reference's operator on the host cores ----
    cpu = None
    if not args.no_cpu:
        from oracle import plexus_oracle as po

        a_cpu = torch.sparse_csr_tensor(g.rowptr.cpu(), g.col.cpu(), g.val.cpu(), size=g.shape)
        h_cpu = S.normal_features(n, d_main, dev, seed=d_main, dtype=dtype).float().cpu()  # bf16 config: fp32 math on bf16-rounded inputs
        po.spmm(a_cpu, h_cpu)  # warm-up
        reps = 2
        t2 = time.time()
        for _ in range(reps):
            y_cpu = po.spmm(a_cpu, h_cpu)
        cpu_s = (time.time() - t2) / reps
        # the same product on the GPU must agree with it
        y_gpu = ops.spmm(a, h_cpu.to(dev).to(dtype)).float().cpu()
        err = ((y_gpu.double() - y_cpu.double()).abs().max() / y_cpu.double().abs().max()).item()
        cpu = {"value": dom["alg_bytes"] / cpu_s / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
               "sample": "the whole SpMM A.H of the workload at D=%d (torch.sparse.mm, fp32, %d timed runs)" % (d_main, reps),
               "ms": cpu_s * 1e3, "GFLOPs": 2.0 * nnz * d_main / cpu_s / 1e9, "host_cpus": os.cpu_count(),
               "max_rel_err_gpu_vs_cpu": err}
        print("# cpu: %.1f ms per SpMM on %d threads, gpu-vs-cpu max rel err %.2e" % (cpu_s * 1e3, cpu["cores"], err),
              file=sys.stderr, flush=True)
        del y_cpu, y_gpu, h_cpu
        if not (args.no_cpu_epoch or args.spmm_only):
            # one whole epoch of the reference's operator chain on the host (fp32; the bf16 configuration runs
            # fp32 math there too, without dropout): forward, loss, backward, AdamW over weights and features
            at_cpu = torch.sparse_csr_tensor(g.rowptr_t.cpu(), g.col_t.cpu(), g.val_t.cpu(), size=(g.shape[1], g.shape[0]))
            x_cpu = S.normal_features(n, dims[0], dev, seed=1).cpu()
            y_lab = S.uniform_labels(n, dims[-1], dev, seed=2).cpu()
            t3 = time.time()
            cpu_losses, _, _ = po.train_epochs(x_cpu, [w.clone() for w in S.glorot_weights(dims, seed=0)], dims, [(a_cpu, at_cpu)],
                                               y_lab, n, dims[-1], epochs=1)
            cpu["epoch_ms"] = (time.time() - t3) * 1e3
            cpu["epoch_sample"] = "one epoch (forward, loss, backward, AdamW) of the same workload, fp32, timed once without warm-up"
            cpu["epoch_first_loss"] = cpu_losses[0]
            print("# cpu: %.0f ms per epoch, first loss %.4f (gpu first loss %.4f)" % (cpu["epoch_ms"], cpu_losses[0], losses[0] if losses else float("nan")),
                  file=sys.stderr, flush=True)

    line = {
        "metric": "SpMM HBM GB/s (% of peak) + GCN fwd+bwd epoch ms on 1 MI355X",
        "value": dom["alg_GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": epoch_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if bf16 else "f32",
        "data": "synthetic",
        "config": {"workload": "config %d: 3-layer GCN %s on a Chung-Lu(2.1) graph, N=%d, nnz=%d "
                               "(value = SpMM A.H at D=%d; step = one training epoch incl. AdamW%s)"
                               % (args.config, "-".join(str(d) for d in dims), n, nnz, d_main,
                                  ", bf16 storage, fp32 accumulate, dropout 0.5" if bf16 else ""),
                   "nodes": n, "nnz": nnz, "max_row_nnz": stats["max_row_nnz"], "scale": args.scale,
                   "split_rows": a.n_long_rows, "segments": a.n_segments},
        "spmm_ms": dom["ms"],
        "spmm_pct_of_hbm_peak": 100.0 * dom["alg_GBps"] / HBM_PEAK_GBPS,
        "spmm_GFLOPs": dom["GFLOPs"],
        "spmm_gather_model_GBps": dom["gather_GBps"],
        "random_gather_ceiling": gather_ceiling,
        "spmm_D%d" % d_side: spmm[d_side],
        "prep_ms": {"narrow_indices_and_plan": prep_plan_ms, "device_transpose_and_plan": prep_transpose_ms,
                    "narrow_indices_and_plan_first_call": prep_plan_first_ms, "device_transpose_and_plan_first_call": prep_transpose_first_ms,
                    "gcn_norm_from_edge_list": prep_norm_ms, "double_permutation": prep_perm_ms},
        "epoch_ms": epoch_ms,
        "epoch_ms_transform_first_option": epoch_ms_tf,
        "loss_first_last": [losses[0], losses[-1]] if losses else None,
        # the dominant kernel: the row kernel of the SpMM (all of the product where the plan has no hub pass)
        "roofline": {"bound": "hbm", "achieved": (parts["row_kernel"] if parts else dom)["alg_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": (parts["row_kernel"] if parts else dom)["alg_GBps"] / HBM_PEAK_GBPS,
                     "traffic": None if bf16 else measured_spmm_traffic(n, nnz, d_main)[0],
                     "traffic_source": None if bf16 else measured_spmm_traffic(n, nnz, d_main)[1],
                     "kernel": "spmm_csr_kernel (A.H, D=%d, %s%s)" % (d_main, "bf16" if bf16 else "fp32",
                                                                       ", the rows outside the hub pass" if parts else ""),
                     "alg_bytes_per_launch": (parts["row_kernel"] if parts else dom)["alg_bytes"],
                     "avg_launch_ms": (parts["row_kernel"] if parts else dom)["ms"]},
        "spmm_parts": parts,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the CLUSTEN hot path on one MI355X.

A step is one pass of the forward hot path over one batch of synthetic input at the AFF-Tiny
stage-1 shape (BASELINE.json configs[2], stage 1: B128, H2, N3136, head dim 32, 48 neighbours,
fp32; WF 3136 -> 784 tokens, 64 channels, 4 inner channels): one QK launch, one AV launch, one WF
launch through the C ABI, inputs resident in HBM.  `value` is the algorithmic bytes of the three ops
(every input read once, every output written once, int64 neighbour lists) divided by the time of a
step.  The three kernels take a third of the step each, so the `roofline` object prices the step: its
`frac` is `value` / 8 TB/s; `kernels` lists the three kernels with the median and the minimum of at
least 50 per-launch HIP-event timings (after at least 10 untimed launches, whatever --steps says), and
`roofline.lowest_kernel` names the one furthest below the peak.  `parity` compares the three outputs
of the headline tensors with the gather oracle on batch elements 0, 63 and 127 and repeats the
comparison bit for bit on integer-valued data; `replay_probe` times the same three kernels compiled
without their arithmetic (same loads, LDS traffic and stores; libclusten_probe.so) in the same
interleaved pass; `cpu_baseline` is the PyTorch gather oracle timed on the host cores on a batch slice
of the same workload, `config0_cpu` the reference's own CPU-runnable configuration timed in full on
both sides.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

The other stages and configurations are timed too and land under "other_configs"; `--quick` leaves
them (and the images/s leg's GEMM tuning) out.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "ml-autofocusformer_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch at the headline workload, from `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE`
# runs of `bench.py --only {qk,av,wf}`, each counter scaled by what it reads for the copy probe of known
# size; see profiles/pmc_hbm_traffic_qk_av_wf_tiny_stage1.md, which names the source revision the
# counters were read at.  A constant of that run, not a measurement of this one: TRAFFIC_MEASURED says when.
MEASURED_TRAFFIC_BYTES = {"qk": 359.59e6 + 154.14e6, "av": 411.70e6 + 102.76e6, "wf": 218.48e6 + 102.76e6}
TRAFFIC_MEASURED = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, see profiles/pmc_hbm_traffic_qk_av_wf_tiny_stage1.md"


def _time_kernels(fns, steps, warmup):
    """Run the launch closures `fns` back to back for warmup + steps steps on the current stream, twice.

    The first timed pass has one event before and one after its `steps` steps and nothing between the launches:
    its duration is the throughput figure.  The second pass records an event after every launch (a marker on
    the stream that costs a few microseconds of gap per launch) for the per-kernel figures.
    Returns (ms per step of the first pass, [median ms per launch of each closure], host wall ms per step,
    [minimum ms per launch of each closure])."""
    import torch

    for _ in range(warmup):
        for fn in fns:
            fn()
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    begin.record()
    for _ in range(steps):
        for fn in fns:
            fn()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    region_ms = begin.elapsed_time(end)

    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(len(fns) + 1)] for _ in range(steps)]
    for s in range(steps):
        marks[s][0].record()
        for i, fn in enumerate(fns):
            fn()
            marks[s][i + 1].record()
    torch.cuda.synchronize()
    samples = [sorted(marks[s][i].elapsed_time(marks[s][i + 1]) for s in range(steps)) for i in range(len(fns))]
    med = [(x[(len(x) - 1) // 2] + x[len(x) // 2]) / 2 for x in samples]
    return region_ms / steps, med, wall_ms / steps, [x[0] for x in samples]


def _cpu_baseline(attn_case, wf_case, full_bytes, full_batch, slice_b=32, budget_s=12.0):
    """The gather oracle on the host cores, on a batch slice of the same inputs: about `budget_s`
    seconds of CPU work."""
    import torch
    from oracle import clusten_oracle as oracle

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    q, k, v, idx = (t[:slice_b] for t in (attn_case.query, attn_case.key, attn_case.value, attn_case.nbhd_idx))
    w, f, widx = (t[:slice_b] for t in (wf_case.weights, wf_case.feat, wf_case.nbhd_idx))

    def one_pass(attn):
        oracle.qk_gather_chunked(q, k, idx)
        oracle.av_gather_chunked(attn, v, idx)
        oracle.wf_gather_chunked(w, f, widx)

    attn = torch.softmax(oracle.qk_gather_chunked(q, k, idx), dim=-1)   # the AV input
    t0 = time.perf_counter()
    one_pass(attn)                                                       # warm-up, and a first estimate
    est = time.perf_counter() - t0
    reps = max(3, min(50, int(budget_s / max(est, 1e-3))))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        one_pass(attn)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    slice_bytes = full_bytes * slice_b / full_batch
    return {
        "value": round(slice_bytes / med / 1e9, 3),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "PyTorch gather oracle (batch chunks of 4), QK+AV+WF forward on a batch slice of %d of %d (same "
                  "tensors), median of %d passes, %.2f s per pass, %.1f s in all; a baseline, not the target"
                  % (slice_b, full_batch, reps, med, sum(times)),
    }


def _parity(acase, wcase, attn_dev, dev_attn_tensors, dw, picks=(0, 63, 127)):
    """The three outputs at the headline tensors against the gather oracle on the host, on the batch elements `picks`
    (outside every timed region): max |x - ref| / max |ref| per operator, and the same three comparisons bit for bit on
    integer-valued data of the same shapes and lists (sums of products of small integers are exact in fp32)."""
    import torch
    from clusten import _native
    from oracle import clusten_oracle as oracle

    q, k, v, idx = dev_attn_tensors
    picks = [b for b in picks if b < q.shape[0]]
    sel = torch.tensor(picks)
    dsel = sel.to(q.device)
    out = {"batch_elements": picks, "tolerance_fp32": 1e-5}
    got_qk = _native.qk_forward(q, k, idx).index_select(0, dsel)
    got_av = _native.av_forward(attn_dev, v, idx).index_select(0, dsel)
    got_wf = _native.wf_forward(dw.weights, dw.feat, dw.nbhd_idx).index_select(0, dsel)
    a_host = attn_dev.index_select(0, dsel).cpu()
    hq, hk, hv, hidx = (t.index_select(0, sel) for t in (acase.query, acase.key, acase.value, acase.nbhd_idx))
    hw, hf, hwidx = (t.index_select(0, sel) for t in (wcase.weights, wcase.feat, wcase.nbhd_idx))
    out["qk_rel_err"] = float("%.3g" % oracle.rel_err(got_qk, oracle.qk_gather_chunked(hq, hk, hidx)))
    out["av_rel_err"] = float("%.3g" % oracle.rel_err(got_av, oracle.av_gather_chunked(a_host, hv, hidx)))
    out["wf_rel_err"] = float("%.3g" % oracle.rel_err(got_wf, oracle.wf_gather_chunked(hw, hf, hwidx)))
    gen = torch.Generator().manual_seed(4242)
    ints = lambda shape, lo, hi: torch.randint(lo, hi, shape, generator=gen).float()
    iq, ik, iv = ints(hq.shape, -8, 9), ints(hk.shape, -8, 9), ints(hv.shape, -8, 9)
    ia = ints(a_host.shape, 0, 5)
    iw, ife = ints(hw.shape, 0, 5), ints(hf.shape, -8, 9)
    dev = q.device
    didx, dwidx = hidx.to(dev), hwidx.to(dev)
    exact = {
        "qk": torch.equal(_native.qk_forward(iq.to(dev), ik.to(dev), didx).cpu(), oracle.qk_gather_chunked(iq, ik, hidx)),
        "av": torch.equal(_native.av_forward(ia.to(dev), iv.to(dev), didx).cpu(), oracle.av_gather_chunked(ia, iv, hidx)),
        "wf": torch.equal(_native.wf_forward(iw.to(dev), ife.to(dev), dwidx).cpu(), oracle.wf_gather_chunked(iw, ife, hwidx)),
    }
    out["integer_data_bit_exact"] = exact
    out["ok"] = bool(all(exact.values()) and max(out["qk_rel_err"], out["av_rel_err"], out["wf_rel_err"]) <= 1e-5)
    return out


def _config0(steps=200):
    """Configuration 0 (the reference's CPU-runnable case: QK forward, B2 H2 N1024 C32 M48 fp32) timed in full on the
    host cores (gather oracle, 3 untimed + 10 timed calls, median) and through the HIP kernel on the same tensors."""
    import torch
    import workloads as wl
    from clusten import _native
    from oracle import clusten_oracle as oracle

    case = wl.config0()
    B, H, N, C = case.query.shape
    M = case.nbhd_idx.shape[-1]
    nbytes = wl.attn_bytes(B, H, N, C, M, 4)
    torch.set_num_threads(os.cpu_count() or 1)
    times = []
    for i in range(13):
        t0 = time.perf_counter()
        ref = oracle.qk_gather(case.query, case.key, case.nbhd_idx)
        if i >= 3:
            times.append(time.perf_counter() - t0)
    times.sort()
    cpu_s = times[len(times) // 2]
    d = case.to("cuda")
    got = _native.qk_forward(d.query, d.key, d.nbhd_idx)
    err = oracle.rel_err(got, ref)
    _, per, _, _ = _time_kernels([lambda: _native.qk_forward(d.query, d.key, d.nbhd_idx)], steps, 10)
    return {"shape": "QK forward B%d H%d N%d C%d M%d fp32" % (B, H, N, C, M), "algorithmic_bytes": nbytes,
            "cpu_ms": round(cpu_s * 1e3, 3), "cpu_GBps": round(nbytes / cpu_s / 1e9, 3),
            "cpu_cores": torch.get_num_threads(), "cpu_calls": "3 untimed + 10 timed, median",
            "gpu_us": round(per[0] * 1e3, 2), "gpu_GBps": round(nbytes / per[0] / 1e6, 1),
            "gpu_note": "2.6 MB: the launch, not the memory system, is what this size measures",
            "rel_err_gpu_vs_cpu": float("%.3g" % err)}


def _stream_gather_interference(tiles=50176, gathers=24, reps=20):
    """How far the device overlaps an operator's two kinds of traffic: streams from / to memory (5 KiB in, 3 KiB out per
    tile) and gathers that hit the L2 (24 KiB per tile inside 800 KB windows shared by 392 tiles — the QK shape), alone
    and together, without arithmetic.  The streams rotate over four buffers so that they come from memory."""
    import torch
    import probe

    sets = 4
    ins = [torch.empty(tiles * 5120, dtype=torch.uint8, device="cuda").random_(0, 255) for _ in range(sets)]
    outs = [torch.empty(tiles * 3072, dtype=torch.uint8, device="cuda") for _ in range(sets)]
    rows = torch.empty((tiles + 391) // 392 * 3136 * 256, dtype=torch.uint8, device="cuda").random_(0, 255)
    res = {}
    for name, mode in (("streams_us", 1), ("gathers_us", 2), ("both_us", 3)):
        turn = [0]

        def one():
            i = turn[0] % sets
            turn[0] += 1
            probe.stream_gather_probe(ins[i], outs[i], rows, tiles, gathers, 3136, 392, mode)

        _, per, _, _ = _time_kernels([one], reps, 4)
        res[name] = round(per[0] * 1e3, 1)
    res["stream_bytes"] = tiles * 8192
    res["gather_bytes"] = tiles * gathers * 1024
    res["streams_GBps"] = round(res["stream_bytes"] / res["streams_us"] / 1e3, 1)
    res["gathers_GBps"] = round(res["gather_bytes"] / res["gathers_us"] / 1e3, 1)
    res["both_over_sum"] = round(res["both_us"] / (res["streams_us"] + res["gathers_us"]), 3)
    return res


def _copy_bandwidth(nbytes=1 << 30, reps=20):
    import torch
    import probe

    src = torch.empty(nbytes // 4, dtype=torch.float32, device="cuda").normal_()
    dst = torch.empty_like(src)
    for _ in range(3):
        probe.copy_probe(src, dst)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        probe.copy_probe(src, dst)
    e1.record()
    torch.cuda.synchronize()
    return 2 * nbytes * reps / (e0.elapsed_time(e1) * 1e-3) / 1e9


def _bench_attn(case, steps, warmup, dtype=None):
    import torch
    import workloads as wl
    from clusten import _native

    d = case.to("cuda")
    q, k, v = d.query, d.key, d.value
    attn = torch.softmax(_native.qk_forward(q, k, d.nbhd_idx).float(), dim=-1).to(q.dtype)
    B, H, N, C = q.shape
    M = d.nbhd_idx.shape[-1]
    nbytes = wl.attn_bytes(B, H, N, C, M, q.element_size())
    # small shapes: rotate among copies of the inputs so that a launch never finds its data in the 256 MB
    # memory-side cache (inputs of one QK + AV pair are about 1.7 x nbytes)
    copies = max(1, min(16, int(700e6 // (1.7 * nbytes)) + 1))
    sets = [(q, k, v, d.nbhd_idx, attn)] + [tuple(t.clone() for t in (q, k, v, d.nbhd_idx, attn)) for _ in range(copies - 1)]
    turn = [0, 0]

    def qk():
        a = sets[turn[0] % copies]
        turn[0] += 1
        return _native.qk_forward(a[0], a[1], a[3])

    def av():
        a = sets[turn[1] % copies]
        turn[1] += 1
        return _native.av_forward(a[4], a[2], a[3])

    _, per, _, _ = _time_kernels([qk, av], steps, warmup)
    return {"shape": "B%d H%d N%d C%d M%d %s" % (B, H, N, C, M, str(q.dtype).replace("torch.", "")),
            "qk_us": round(per[0] * 1e3, 1), "qk_GBps": round(nbytes / per[0] / 1e6, 1),
            "av_us": round(per[1] * 1e3, 1), "av_GBps": round(nbytes / per[1] / 1e6, 1), "bytes_each": nbytes,
            "input_sets_rotated": copies}


def _bench_backward(acase, wcase, steps, warmup):
    """Backward of the three operators at one shape: microseconds per call (both gradients of each operator)."""
    import torch
    from clusten import _native

    d, w = acase.to("cuda"), wcase.to("cuda")
    q, k, v, idx = d.query, d.key, d.value, d.nbhd_idx
    attn = torch.softmax(_native.qk_forward(q, k, idx).float(), dim=-1).to(q.dtype)
    d_attn = torch.randn_like(attn)
    d_feat = torch.randn_like(q)
    d_out = torch.randn(w.weights.shape[0], w.weights.shape[1], w.weights.shape[3], w.feat.shape[2],
                        dtype=w.feat.dtype, device="cuda")
    pairs = _native.cluster_pairs(idx)     # what a harness builds once per stage and hands to every layer's backward
    fns = [lambda: _native.qk_backward(d_attn, q, k, idx),
           lambda: _native.av_backward(d_feat, attn, v, idx),
           lambda: _native.wf_backward(d_out, w.weights, w.feat, w.nbhd_idx)]
    if pairs is not None:
        fns += [lambda: _native.qk_backward(d_attn, q, k, idx, pairs=pairs),
                lambda: _native.av_backward(d_feat, attn, v, idx, pairs=pairs)]
    _, per, _, _ = _time_kernels(fns, steps, warmup)
    out = {"qk_backward_us": round(per[0] * 1e3, 1), "av_backward_us": round(per[1] * 1e3, 1),
           "wf_backward_us": round(per[2] * 1e3, 1)}
    if pairs is not None:
        out["qk_backward_with_the_callers_pair_lists_us"] = round(per[3] * 1e3, 1)
        out["av_backward_with_the_callers_pair_lists_us"] = round(per[4] * 1e3, 1)
    return out


def _bench_wf(case, steps, warmup):
    import workloads as wl
    from clusten import _native

    d = case.to("cuda")
    B, Nout, M, IC = d.weights.shape
    N, C = d.feat.shape[1], d.feat.shape[2]
    nbytes = wl.wf_bytes(B, N, Nout, C, M, IC, d.feat.element_size())
    copies = max(1, min(16, int(700e6 // nbytes) + 1))   # see _bench_attn
    sets = [(d.weights, d.feat, d.nbhd_idx)] + [tuple(t.clone() for t in (d.weights, d.feat, d.nbhd_idx))
                                                for _ in range(copies - 1)]
    turn = [0]

    def wf():
        a = sets[turn[0] % copies]
        turn[0] += 1
        return _native.wf_forward(*a)

    _, per, _, _ = _time_kernels([wf], steps, warmup)
    return {"shape": "B%d N%d->%d C%d M%d IC%d %s" % (B, N, Nout, C, M, IC, str(d.feat.dtype).replace("torch.", "")),
            "wf_us": round(per[0] * 1e3, 1), "wf_GBps": round(nbytes / per[0] / 1e6, 1), "bytes": nbytes,
            "input_sets_rotated": copies}


def _bench_local_attention(B, H, N, dtype, steps, warmup, cluster=8, views=False, random_bias_rows=False):
    """The one-kernel local attention (QK, bias, mask, blank token, softmax, AV) of one block at a stage's shape on
    lists built by the model's clustering, with the plan of the stage; microseconds per call."""
    import torch
    import workloads as wl
    from clusten import _native

    mcase = wl.attn_case("model", 29, B=B, H=H, N=N, C=32, M=6 * cluster, lists="random")
    mcase.nbhd_idx, pe_idx, rows = wl.model_built_geometry(B, N, wl.generator(29), cluster=cluster, nnc=6)
    mcase = mcase.to("cuda")
    cidx = (mcase.nbhd_idx[:, :, ::cluster] // cluster).to(torch.int32).contiguous()
    gen = torch.Generator().manual_seed(1029)
    if random_bias_rows:
        pe_idx = torch.randint(rows, pe_idx.shape, generator=gen)
    pe_idx = pe_idx.cuda()
    q, k, v = (t.to(dtype) for t in (mcase.query, mcase.key, mcase.value))
    if views:
        # the operands as a model's projections leave them: q a (B,N,H,C) tensor, k and v the two halves of a
        # (B,N,H,2,C) tensor (models/aff_transformer.py:112-118), all three handed over as permuted views
        kv = torch.stack([k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3)], dim=3).contiguous()      # (B,N,H,2,C)
        q = q.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
        k, v = kv[:, :, :, 0].permute(0, 2, 1, 3), kv[:, :, :, 1].permute(0, 2, 1, 3)
    table = torch.randn(rows, H, generator=gen).to(dtype).cuda()
    blank_k, blank_v = torch.randn(H * 32, generator=gen).cuda(), torch.randn(H * 32, generator=gen).cuda()
    plan = _native.cluster_attention_plan(cidx, pe_idx, None)
    _, per, _, per_min = _time_kernels([lambda: _native.cluster_attention(q, k, v, None, table, None, None, blank_k,
                                                                          blank_v, plan=plan)], steps, warmup)
    nbytes = 4 * q.numel() * q.element_size() + plan.numel()
    return {"shape": "B%d H%d N%d C32 M%d %s, model-built lists and position indices, planned%s%s" % (
                B, H, N, 6 * cluster, str(dtype).replace("torch.", ""), ", q / k / v as views of the projections" if views else "",
                ", position indices drawn uniformly from the table instead" if random_bias_rows else ""),
            "median_us": round(per[0] * 1e3, 1), "min_us": round(per_min[0] * 1e3, 1),
            "bytes_q_k_v_out_plan": nbytes, "GBps": round(nbytes / per[0] / 1e6, 1)}


def _aff_tiny_throughput(batch=128, warmup=50, timed=30, tune_gemms=True):
    """Images/s of the AFF-Tiny classifier at 224x224 (random weights, N(0,1) images, fp16 autocast, eval mode, no_grad),
    timed like the reference's `throughput` (main.py:343-354: 50 untimed and 30 timed forwards), and the share
    of one forward spent in each operator, measured in a separate pass with stream events around the calls."""
    import torch
    from types import SimpleNamespace
    from aff import model as aff_model

    torch.manual_seed(0)
    spans = {}

    def timed_call(name, fn):
        def call(*a, **kw):
            if not spans.get("on"):
                return fn(*a, **kw)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = fn(*a, **kw)
            e1.record()
            spans.setdefault(name, []).append((e0, e1))
            return out
        return call

    real = aff_model.default_ops()
    ops = SimpleNamespace(**vars(real))
    ops.qk, ops.av, ops.wf = timed_call("qk", real.qk), timed_call("av", real.av), timed_call("wf", real.wf)
    ops.attn_softmax = timed_call("bias+mask+blank+softmax", real.attn_softmax)
    ops.qk_clusters, ops.av_clusters = timed_call("qk", real.qk_clusters), timed_call("av", real.av_clusters)
    ops.cluster_attention = timed_call("qk+bias+mask+blank+softmax+av (one kernel)", real.cluster_attention)
    ops.dense_attention = timed_call("global attention (one kernel)", real.dense_attention)
    ops.layer_norm = timed_call("layer_norm", real.layer_norm)
    ops.add_layer_norm = timed_call("layer_norm", real.add_layer_norm)
    ops.linear = timed_call("small Linear layers (+GELU) of stage 1", real.linear)
    ops.merge_weights = timed_call("merge_weights", real.merge_weights)
    ops.channel_affine_gelu = timed_call("patch embedding epilogues", real.channel_affine_gelu)
    net = aff_model.aff_tiny(ops=ops).cuda().eval()
    for layer in net.layers:
        layer.neighbourhoods = timed_call("clustering+knn", layer.neighbourhoods)
        if layer.downsample is not None:
            layer.downsample.select = timed_call("merge_select", layer.downsample.select)
    x = torch.randn(batch, 3, 224, 224, device="cuda")

    def forward():
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.float16):
            return net(x)

    for _ in range(warmup):
        forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(timed):
        forward()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0

    # the same forward recorded into a HIP graph and replayed (the input copy into the recording's buffer included);
    # before the recording PyTorch's TunableOp picks, per Linear shape, the fastest of the GEMM solutions rocBLAS and
    # hipBLASLt offer (a few seconds, results kept only for this process; the logits are checked against the
    # untuned forward)
    gemm_tuning = "library defaults"
    try:
        if not tune_gemms:
            raise RuntimeError("switched off")
        import tempfile
        import torch.cuda.tunable as tunable
        want = forward().float()
        tunable.set_filename(os.path.join(tempfile.gettempdir(), "clusten_bench_tunableop.csv"))
        tunable.enable(True)
        tunable.tuning_enable(True)
        forward()
        torch.cuda.synchronize()
        tunable.tuning_enable(False)
        got = forward().float()
        if float((got - want).abs().max()) <= 1e-2 * float(want.abs().max()):
            gemm_tuning = "PyTorch TunableOp, tuned in this process before the recording"
        else:
            tunable.enable(False)
    except Exception as exc:  # noqa: BLE001 - an optional speed-up: report and go on without it
        if tune_gemms:
            gemm_tuning = "library defaults (TunableOp unavailable: %s)" % type(exc).__name__
    launch = "one HIP graph replay per forward (aff.model.CapturedForward)"
    try:
        recorded = aff_model.CapturedForward(net, x)
        x2 = torch.randn_like(x)
        for _ in range(warmup):
            recorded(x2)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(timed):
            recorded(x2)
        torch.cuda.synchronize()
        dt_graph = time.perf_counter() - t0
        del recorded
    except Exception as exc:  # noqa: BLE001 - the eager figure stands when the recording is not possible
        launch = "eager launches (recording into a HIP graph failed: %s)" % type(exc).__name__
        dt_graph = dt
    try:
        tunable.enable(False)
    except Exception:  # noqa: BLE001
        pass

    spans["on"] = True
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    forward()
    e1.record()
    torch.cuda.synchronize()
    total = e0.elapsed_time(e1)
    share = {k: round(sum(a.elapsed_time(b) for a, b in v) / total, 4) for k, v in spans.items() if k != "on"}
    share["everything_else"] = round(1.0 - sum(share.values()), 4)
    return {"img_per_s": round(timed * batch / dt_graph, 1), "ms_per_batch": round(dt_graph / timed * 1e3, 2),
            "launch": launch,
            "gemm_selection": gemm_tuning,
            "eager_img_per_s": round(timed * batch / dt, 1), "eager_ms_per_batch": round(dt / timed * 1e3, 2),
            "batch": batch, "warmup": warmup, "timed": timed,
            "dtype": "fp16 autocast (attention: one fp16 kernel per layer, fp32 sums; WF fp32)",
            "inference_path": "16-bit weight copies, position-bias tables and merge-weight tables kept between "
                              "forwards; layer norm (with the residual addition ahead of it), merge centres and the rows at them, merge weights, kNN, token "
                              "ranking, neighbour lists, local and global attention, the small Linear layers of stage 1 "
                              "and the patch embedding's epilogues through the HIP library's optional entry points",
            "share_of_forward": share}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--full", action="store_true", help="(default now) also time the other stages and configurations")
    ap.add_argument("--quick", action="store_true",
                    help="headline only: leave out the other configurations and the GEMM tuning of the images/s leg")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU legs (the baseline and configuration 0)")
    ap.add_argument("--no-e2e", action="store_true", help="skip the AFF-Tiny images/s leg")
    ap.add_argument("--no-parity", action="store_true",
                    help="skip the parity leg (its small launches would enter a profiler's per-kernel averages)")
    ap.add_argument("--e2e-only", action="store_true", help="run just the AFF-Tiny images/s leg")
    ap.add_argument("--no-gemm-tuning", action="store_true",
                    help="images/s leg: keep the GEMM libraries' default solutions (no TunableOp pass; for profilers)")
    ap.add_argument("--batch", type=int, default=None,
                    help="batch size of the --only wf-cfg3* / ca-* profiler legs (default: the configuration's own)")
    ap.add_argument("--random-bias-rows", action="store_true",
                    help="ca-* legs: position indices drawn uniformly from the table (every slot another cache line) "
                         "instead of the offsets between the tokens' positions")
    ap.add_argument("--only", choices=("qk", "av", "wf", "copy", "bwd", "bwd-model", "replay-qk", "replay-av", "replay-wf",
                                       "interference", "wf-cfg3", "wf-cfg3-f32", "ca-s1-f16", "ca-s1-f32", "ca-s2-f16",
                                       "ca-s3-f16", "ca-384-f16", "ca-s1-f16-views", "ca-s2-f16-views", "ca-s3-f16-views"),
                    default=None,
                    help="launch just this kernel warmup+steps times (for profilers); prints a short JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the hot path shards trivially over the batch axis and "
                 "needs no exchange); --gpus %d is not supported, use --gpus 1." % args.gpus)

    import torch
    import probe
    import workloads as wl
    from clusten import _native

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the CLUSTEN kernels have no CPU path.")
    _native.load()
    torch.cuda.set_device(0)
    if args.e2e_only:
        print(json.dumps({"aff_tiny_224": _aff_tiny_throughput(tune_gemms=not args.no_gemm_tuning)}), flush=True)
        return

    if args.only == "interference":
        print(json.dumps({"only": "interference", **_stream_gather_interference()}), flush=True)
        return
    if args.only in ("wf-cfg3", "wf-cfg3-f32"):   # configuration 3's WF (9216 -> 2304 tokens, C = 128), bf16 or fp32
        dt = torch.bfloat16 if args.only == "wf-cfg3" else torch.float32
        print(json.dumps({"only": args.only, "launches": 2 * (args.steps + args.warmup),
                          **_bench_wf(wl.config3_wf(dtype=dt, B=args.batch or 64), args.steps, args.warmup)}), flush=True)
        return
    if args.only == "ca-384-f16":   # ... at the first stage of a 384 x 384 model: clusters of 24, 144 neighbours
        print(json.dumps({"only": args.only, "launches": 2 * (args.steps + args.warmup),
                          **_bench_local_attention(args.batch or 16, 4, 9216, torch.float16, args.steps, args.warmup,
                                                   cluster=24, random_bias_rows=args.random_bias_rows)}), flush=True)
        return
    if args.only and args.only.startswith("ca-"):   # the one-kernel local attention at a stage's shape, with its plan
        stage, dt = int(args.only[4]), (torch.float16 if "f16" in args.only else torch.float32)
        H, N = {1: (2, 3136), 2: (4, 784), 3: (8, 196)}[stage]
        print(json.dumps({"only": args.only, "launches": 2 * (args.steps + args.warmup),
                          **_bench_local_attention(args.batch or 128, H, N, dt, args.steps, args.warmup,
                                                   views=args.only.endswith("-views"),
                                                   random_bias_rows=args.random_bias_rows)}), flush=True)
        return
    B = 128
    acase = wl.config2_attn(1, B=B)
    wcase = wl.config2_wf(1, IC=4, B=B)
    da, dw = acase.to("cuda"), wcase.to("cuda")
    q, k, v, idx = da.query, da.key, da.value, da.nbhd_idx
    attn = torch.softmax(_native.qk_forward(q, k, idx), dim=-1)
    H, N, C, M = q.shape[1], q.shape[2], q.shape[3], idx.shape[2]
    qk_bytes = wl.attn_bytes(B, H, N, C, M, 4)
    wf_bytes = wl.wf_bytes(B, wcase.feat.shape[1], wcase.weights.shape[1], wcase.feat.shape[2], M, 4, 4)
    total_bytes = 2 * qk_bytes + wf_bytes

    fns = [lambda: _native.qk_forward(q, k, idx),
           lambda: _native.av_forward(attn, v, idx),
           lambda: _native.wf_forward(dw.weights, dw.feat, dw.nbhd_idx)]
    # the same kernels without their arithmetic (same loads, LDS traffic and stores): see include/clusten_probe.h
    replay_fns = [lambda: probe.qk_forward_replay(q, k, idx),
                  lambda: probe.av_forward_replay(attn, v, idx),
                  lambda: probe.wf_forward_replay(dw.weights, dw.feat, dw.nbhd_idx)]
    torch.cuda.synchronize()
    if args.only == "bwd-model":  # the same on lists as the model builds them (whole clusters, nearest first)
        mcase = wl.attn_case("model", 29, B=B, H=2, N=3136, C=32, lists="model_built")
        print(json.dumps({"only": "bwd-model", "launches": args.steps + args.warmup,
                          **_bench_backward(mcase, wcase, args.steps, args.warmup)}), flush=True)
        return
    if args.only == "bwd":  # the three backward operators, for profilers
        print(json.dumps({"only": "bwd", "launches": args.steps + args.warmup,
                          **_bench_backward(acase, wcase, args.steps, args.warmup)}), flush=True)
        return
    if args.only:
        if args.only == "copy":  # a plain copy of known traffic, to calibrate a profiler's byte counters
            src = torch.empty(qk_bytes // 8, dtype=torch.float32, device="cuda").normal_()
            dst = torch.empty_like(src)
            one, nbytes = (lambda: probe.copy_probe(src, dst)), 2 * src.numel() * 4
        elif args.only.startswith("replay-"):
            # interleaved with the other two real kernels, as in the default pass: the probe's inputs come from HBM
            i = ("qk", "av", "wf").index(args.only[7:])
            trio = list(fns)
            trio[i] = replay_fns[i]
            _, per3, _, _ = _time_kernels(trio, args.steps, args.warmup)
            print(json.dumps({"only": args.only, "launches": args.steps + args.warmup,
                              "avg_us": round(per3[i] * 1e3, 2)}), flush=True)
            return
        else:
            i = ("qk", "av", "wf").index(args.only)
            one, nbytes = fns[i], (qk_bytes, qk_bytes, wf_bytes)[i]
        _, per, _, _ = _time_kernels([one], args.steps, args.warmup)
        print(json.dumps({"only": args.only, "launches": args.steps + args.warmup, "avg_us": round(per[0] * 1e3, 2),
                          "algorithmic_bytes": nbytes, "achieved_GBps": round(nbytes / per[0] / 1e6, 1)}), flush=True)
        return
    # throughput: exactly --steps steps after --warmup untimed ones; per-kernel figures: at least 10 + 50 launches.
    # A process that has just started runs its first few tens of milliseconds of kernels some 5 % slower (the device's
    # clocks are still rising), so the same measurement is taken twice: `cold_start` is the one right after start-up,
    # `value` the one that follows it, with the device in the state a training or serving loop keeps it in.
    cold_ms, _, _, _ = _time_kernels(fns, args.steps, args.warmup)
    torch.cuda.synchronize()
    ms_per_step, per, wall_ms, per_min = _time_kernels(fns, args.steps, args.warmup)
    torch.cuda.synchronize()
    k_steps, k_warm = max(args.steps, 50), max(args.warmup, 10)
    if (k_steps, k_warm) != (args.steps, args.warmup):
        _, per, _, per_min = _time_kernels(fns, k_steps, k_warm)
        torch.cuda.synchronize()
    _, per_replay, _, _ = _time_kernels(replay_fns, k_steps, k_warm)
    torch.cuda.synchronize()
    # The same step over three sets of tensors taken in turn (lists included), so that no launch finds anything of the
    # step before it in the 256 MB memory-side cache.  Within a step QK and AV share their lists, as in an attention layer.
    sets = [(q, k, v, idx, attn, dw.weights, dw.feat, dw.nbhd_idx)]
    for _ in range(2):
        sets.append(tuple(t.clone() for t in sets[0]))
    turn = [0]

    def _next_set():
        turn[0] += 1

    rot_fns = [lambda: _native.qk_forward(sets[turn[0] % 3][0], sets[turn[0] % 3][1], sets[turn[0] % 3][3]),
               lambda: _native.av_forward(sets[turn[0] % 3][4], sets[turn[0] % 3][2], sets[turn[0] % 3][3]),
               lambda: (_native.wf_forward(sets[turn[0] % 3][5], sets[turn[0] % 3][6], sets[turn[0] % 3][7]), _next_set())]
    rot_ms, rot_per, _, _ = _time_kernels(rot_fns, k_steps, k_warm)
    torch.cuda.synchronize()
    del sets[1:]

    names = ("gather_dot_tile_kernel (QK)", "gather_sum_tile_kernel (AV)", "wf_forward_row_kernel (WF)")
    kbytes = (qk_bytes, qk_bytes, wf_bytes)
    kernels = [{"kernel": n, "median_us": round(t * 1e3, 2), "min_us": round(tm * 1e3, 2), "launches_timed": k_steps,
                "algorithmic_bytes": nb, "measured_hbm_bytes": MEASURED_TRAFFIC_BYTES[key],
                "achieved_GBps": round(nb / t / 1e6, 1), "frac_of_hbm_peak": round(nb / t / 1e6 / HBM_PEAK_GBPS, 4)}
               for n, key, t, tm, nb in zip(names, ("qk", "av", "wf"), per, per_min, kbytes)]
    # The three kernels take a third of the step each, so the roofline object prices the step (the north-star
    # quantity): algorithmic bytes of the three launches over the time of a step.  `kernels` lists all three.
    low = min(range(3), key=lambda i: kbytes[i] / per[i])
    value = total_bytes / ms_per_step / 1e6
    out = {
        "metric": "CLUSTEN QK+AV+WF forward, algorithmic GB/s (AFF-Tiny stage-1 shape)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[2] stage 1: QK+AV+WF(IC=4) forward, B128 H2 N3136 C32 M48 fp32, "
                               "WF 3136->784 C64; cluster-shared windowed lists (QK/AV), 48-nearest lists (WF)",
                   "global_batch": B, "algorithmic_bytes_per_step": total_bytes},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "roofline": {"bound": "hbm", "achieved": round(value, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(value / HBM_PEAK_GBPS, 4),
                     "traffic": sum(MEASURED_TRAFFIC_BYTES.values()), "traffic_source": TRAFFIC_MEASURED,
                     "kernel": "the step: one launch each of " + ", ".join(names),
                     "lowest_kernel": {"kernel": names[low], "frac": kernels[low]["frac_of_hbm_peak"],
                                       "achieved": kernels[low]["achieved_GBps"]}},
        "kernels": kernels,
        "cold_start": {"what": "the same --warmup + --steps measurement taken first, right after the process started",
                       "ms_per_step": round(cold_ms, 4), "GBps": round(total_bytes / cold_ms / 1e6, 1)},
        "rotating_inputs": {"what": "the same step over three sets of tensors taken in turn (lists too): nothing of the "
                                    "step before is in the memory-side cache; QK and AV of a step share their lists",
                            "sets": 3, "ms_per_step": round(rot_ms, 4), "GBps": round(total_bytes / rot_ms / 1e6, 1),
                            "median_us": [round(t * 1e3, 2) for t in rot_per]},
        "parity": None if args.no_parity else _parity(acase, wcase, attn, (q, k, v, idx), dw),
        "replay_probe": {"what": "the same kernels compiled without their matrix instructions (same global loads, LDS "
                                 "accesses and stores; libclusten_probe.so), timed in the same interleaved pass",
                         "kernels": [{"kernel": n, "replay_us": round(r * 1e3, 2), "kernel_us": round(t * 1e3, 2),
                                      "kernel_over_replay": round(t / r, 3)}
                                     for n, t, r in zip(names, per, per_replay)]},
        "host_wall_ms_per_step": round(wall_ms, 4),
        "copy_probe_GBps": round(_copy_bandwidth(), 1),
        "stream_gather_interference": _stream_gather_interference(),
    }
    if not args.no_cpu:
        out["config0_cpu"] = _config0()
    if not args.quick:
        other = {}
        for s in (2, 3, 4):
            other["cfg2_s%d_attn" % s] = _bench_attn(wl.config2_attn(s, B=B), args.steps, args.warmup)
            other["cfg2_s%d_wf_ic4" % s] = _bench_wf(wl.config2_wf(s, IC=4, B=B), args.steps, args.warmup)
        other["cfg2_s1_wf_ic1"] = _bench_wf(wl.config2_wf(1, IC=1, B=B), args.steps, args.warmup)
        other["cfg1_fp32"] = _bench_attn(wl.config1(torch.float32), args.steps, args.warmup)
        other["cfg1_fp16"] = _bench_attn(wl.config1(torch.float16), args.steps, args.warmup)
        other["cfg3_bf16_attn"] = _bench_attn(wl.config3_attn(), args.steps, args.warmup)
        other["cfg3_bf16_wf_ic4"] = _bench_wf(wl.config3_wf(), args.steps, args.warmup)
        # lists built by the model's own clustering of adaptively kept tokens (`workloads.model_built_lists`), and the
        # strips of a regular grid used before that generator existed (fewer distinct clusters per tile: faster)
        other["cfg2_s1_model_built_lists"] = _bench_attn(
            wl.attn_case("model", 29, B=B, H=2, N=3136, C=32, lists="model_built"), args.steps, args.warmup)
        other["cfg2_s1_model_like_lists"] = _bench_attn(
            wl.attn_case("model", 29, B=B, H=2, N=3136, C=32, lists="model"), args.steps, args.warmup)
        mcase = wl.attn_case("model", 29, B=B, H=2, N=3136, C=32, lists="random")
        # the lists with the position indices that go with them: offsets between the tokens' positions, as the model
        # computes them (uniformly drawn indices would make every slot's bias another cache line)
        mcase.nbhd_idx, pe_idx, rows = wl.model_built_geometry(B, 3136, wl.generator(29))
        mcase, pe_idx = mcase.to("cuda"), pe_idx.cuda()
        cidx = (mcase.nbhd_idx[:, :, ::8] // 8).to(torch.int32).contiguous()   # the same lists as cluster numbers
        mattn = torch.softmax(_native.qk_forward(mcase.query, mcase.key, mcase.nbhd_idx), dim=-1)
        _, per_c, _, _ = _time_kernels([lambda: _native.qk_forward_clusters(mcase.query, mcase.key, cidx),
                                     lambda: _native.av_forward_clusters(mattn, mcase.value, cidx)],
                                    args.steps, args.warmup)
        other["cfg2_s1_model_built_lists_as_cluster_numbers"] = {"qk_us": round(per_c[0] * 1e3, 1),
                                                                  "av_us": round(per_c[1] * 1e3, 1)}
        # local attention of one block at the same shape under mixed precision: one kernel against the three
        # operators' kernels with the softmax kernel between them (what the model ran before)
        h16 = lambda t: t.to(torch.float16)
        q16, k16, v16 = h16(mcase.query), h16(mcase.key), h16(mcase.value)
        gen = torch.Generator().manual_seed(1029)
        table = h16(torch.randn(rows, 2, generator=gen)).cuda()
        blank_k, blank_v = torch.randn(64, generator=gen).cuda(), torch.randn(64, generator=gen).cuda()

        def three_kernels():
            a = _native.qk_forward_clusters(q16, k16, cidx)
            p, pb = _native.attn_softmax(a, table, pe_idx, None, query=q16, blank_key=blank_k)
            return _native.av_forward_clusters(p, v16, cidx)

        plan = _native.cluster_attention_plan(cidx, pe_idx, None)   # what a stage builds once for all its layers
        _, per_a, _, _ = _time_kernels([lambda: _native.cluster_attention(q16, k16, v16, cidx, table, pe_idx, None,
                                                                       blank_k, blank_v), three_kernels,
                                     lambda: _native.cluster_attention(q16, k16, v16, None, table, None, None,
                                                                       blank_k, blank_v, plan=plan)],
                                    args.steps, args.warmup)
        fused_bytes = 4 * q16.numel() * 2 + cidx.numel() * 4 + pe_idx.numel() * 8
        other["cfg2_s1_local_attention_fp16_model_built_lists"] = {
            "one_kernel_us": round(per_a[0] * 1e3, 1), "three_kernels_us": round(per_a[1] * 1e3, 1),
            "one_kernel_with_plan_us": round(per_a[2] * 1e3, 1),
            "one_kernel_algorithmic_bytes": fused_bytes, "one_kernel_GBps": round(fused_bytes / per_a[0] / 1e6, 1)}
        # ... and its backward: one kernel for the query side (probabilities recomputed) + the two scatters over sorted
        # pair lists + the bias table's gradient, against the backward functions of the three operators with the
        # softmax kernel's backward between them (pair lists of the stage built once, outside both)
        out16, lse = _native.cluster_attention(q16, k16, v16, None, table, None, None, blank_k, blank_v, plan=plan,
                                               return_lse=True)
        g16 = h16(torch.randn(out16.shape, generator=gen)).cuda()
        pairs = _native.cluster_pairs(mcase.nbhd_idx)
        g_view = g16.view(B, 3136, 2, 32).permute(0, 2, 1, 3)
        probs16, pb16 = _native.attn_softmax(_native.qk_forward_clusters(q16, k16, cidx), table, pe_idx, None, query=q16,
                                             blank_key=blank_k)

        g32, v32 = g_view.float().contiguous(), mcase.value
        def fused_backward():
            dq, p_, ds_, pb_, dsb_ = _native.cluster_attention_backward(q16, k16, v16, g16, out16, lse, plan, table,
                                                                      blank_k, blank_v)
            dv = _native.scatter_rows_by_cluster(p_, g_view, pairs)
            dk = _native.scatter_rows_by_cluster(ds_, q16, pairs)
            return _native.bias_table_grad(ds_, pe_idx, rows), dq, dk, dv

        def operator_backward():
            # (under mixed precision the softmax kernel hands AV fp32 probabilities and the AV Function casts v up)
            d_p, dv = _native.av_backward(g32, probs16, v32, mcase.nbhd_idx)
            d_logit, d_blank = _native.attn_softmax_backward(probs16, pb16, d_p, torch.zeros_like(pb16), torch.float16)
            d_table = _native.bias_table_grad(d_logit, pe_idx, rows)
            return (d_table,) + tuple(_native.qk_backward(d_logit, q16, k16, mcase.nbhd_idx)) + (dv,)

        _, per_b, _, _ = _time_kernels([fused_backward, operator_backward], max(args.steps // 5, 5), 3)
        other["cfg2_s1_local_attention_fp16_backward_model_built_lists"] = {
            "one_kernel_path_us": round(per_b[0] * 1e3, 1), "operator_path_us": round(per_b[1] * 1e3, 1),
            "what": "d_query, d_key, d_value and the bias table's gradient of one block's local attention"}
        del out16, lse, g16, pairs, probs16, pb16, g32, v32
        # the same in fp32 (inference without mixed precision)
        table32 = table.float()

        def three_kernels_fp32():
            a = _native.qk_forward_clusters(mcase.query, mcase.key, cidx)
            p, pb = _native.attn_softmax(a, table32, pe_idx, None, query=mcase.query, blank_key=blank_k)
            return _native.av_forward_clusters(p, mcase.value, cidx)

        _, per_f, _, _ = _time_kernels([lambda: _native.cluster_attention(mcase.query, mcase.key, mcase.value, cidx, table32,
                                                                       pe_idx, None, blank_k, blank_v),
                                     three_kernels_fp32,
                                     lambda: _native.cluster_attention(mcase.query, mcase.key, mcase.value, None, table32,
                                                                       None, None, blank_k, blank_v, plan=plan)],
                                    args.steps, args.warmup)
        fused_bytes32 = 4 * mcase.query.numel() * 4 + cidx.numel() * 4 + pe_idx.numel() * 8
        other["cfg2_s1_local_attention_fp32_model_built_lists"] = {
            "one_kernel_us": round(per_f[0] * 1e3, 1), "three_kernels_us": round(per_f[1] * 1e3, 1),
            "one_kernel_with_plan_us": round(per_f[2] * 1e3, 1),
            "one_kernel_algorithmic_bytes": fused_bytes32, "one_kernel_GBps": round(fused_bytes32 / per_f[0] / 1e6, 1)}
        # ... and its backward in fp32, against the backward functions of the three operators around the softmax's
        out32, lse32 = _native.cluster_attention(mcase.query, mcase.key, mcase.value, None, table32, None, None, blank_k,
                                                 blank_v, plan=plan, return_lse=True)
        gout32 = torch.randn(out32.shape, generator=gen).cuda()
        gview32 = gout32.view(B, 3136, 2, 32).permute(0, 2, 1, 3)
        pairs = _native.cluster_pairs(mcase.nbhd_idx)
        probs32, pb32 = _native.attn_softmax(_native.qk_forward_clusters(mcase.query, mcase.key, cidx), table32, pe_idx,
                                             None, query=mcase.query, blank_key=blank_k)

        def fused_backward_fp32():
            dq, p_, ds_, pb_, dsb_ = _native.cluster_attention_backward(mcase.query, mcase.key, mcase.value, gout32, out32,
                                                                      lse32, plan, table32, blank_k, blank_v)
            dv = _native.scatter_rows_by_cluster(p_, gview32, pairs)
            dk = _native.scatter_rows_by_cluster(ds_, mcase.query, pairs)
            return _native.bias_table_grad(ds_, pe_idx, rows), dq, dk, dv

        def operator_backward_fp32():
            d_p, dv = _native.av_backward(gview32, probs32, mcase.value, mcase.nbhd_idx, pairs=pairs)
            d_logit, d_blank = _native.attn_softmax_backward(probs32, pb32, d_p, torch.zeros_like(pb32), torch.float32)
            d_table = _native.bias_table_grad(d_logit, pe_idx, rows)
            return (d_table,) + tuple(_native.qk_backward(d_logit, mcase.query, mcase.key, mcase.nbhd_idx, pairs=pairs)) + (dv,)

        _, per_g, _, _ = _time_kernels([fused_backward_fp32, operator_backward_fp32], max(args.steps // 5, 5), 3)
        other["cfg2_s1_local_attention_fp32_backward_model_built_lists"] = {
            "one_kernel_path_us": round(per_g[0] * 1e3, 1), "operator_path_us": round(per_g[1] * 1e3, 1),
            "what": "d_query, d_key, d_value and the bias table's gradient of one block's local attention, fp32"}
        del out32, lse32, gout32, gview32, pairs, probs32, pb32
        del mcase, cidx, mattn, q16, k16, v16, pe_idx, plan, table32
        # WF on the lists a merge reads (the members of the nearest clusters of every centre, centres = a sorted
        # quarter of the tokens of a cluster-ordered sequence): consecutive output tokens name mostly the same rows
        def _wf_merge(tag, B_, N_, C_, cluster, steps):
            g_ = wl.generator(33)
            lists = wl.model_built_lists(B_, N_, g_, cluster=cluster, nnc=6)
            centres = torch.stack([torch.randperm(N_, generator=g_)[:N_ // 4].sort().values for _ in range(B_)])
            wc = wl.wf_case(tag, 34, B=B_, N=N_, C=C_, M=lists.shape[2])
            wc.nbhd_idx = lists.gather(1, centres[:, :, None].expand(-1, -1, lists.shape[2])).contiguous()
            return _bench_wf(wc, steps, 5)

        other["cfg2_s1_wf_merge_lists"] = _wf_merge("wf_merge", B, 3136, 64, 8, args.steps)
        other["aff_base_384_stage1_wf_merge_lists"] = _wf_merge("wf_merge_384", 16, 9216, 128, 24, max(args.steps // 2, 5))
        # the first stage of the 384 x 384 models as the reference model builds its lists there: clusters of 24 tokens,
        # the members of the 6 nearest clusters = 144 slots (configs/aff_base_22kto1k_384.yaml:10-11), B = 16
        for dt, tag in ((torch.float32, "fp32"), (torch.bfloat16, "bf16")):
            gen384 = wl.generator(31)
            c384 = wl.attn_case("aff_base_384", 31, B=16, H=4, N=9216, C=32, M=144, dtype=dt, lists="random")
            c384.nbhd_idx, pe384, rows384 = wl.model_built_geometry(16, 9216, gen384, cluster=24, nnc=6)
            other["aff_base_384_stage1_model_lists_%s" % tag] = _bench_attn(c384, max(args.steps // 2, 5), 5)
            if dt == torch.float32:
                # the same lists as (B,N,6) int32 numbers of clusters of 24 rows instead of (B,N,144) int64 rows
                dn = c384.to("cuda")
                cn = (dn.nbhd_idx[:, :, ::24] // 24).to(torch.int32).contiguous()
                pn = torch.softmax(_native.qk_forward(dn.query, dn.key, dn.nbhd_idx), dim=-1)
                _, per_n, _, _ = _time_kernels([lambda: _native.qk_forward_clusters(dn.query, dn.key, cn, cluster_size=24),
                                                lambda: _native.av_forward_clusters(pn, dn.value, cn, cluster_size=24)],
                                               max(args.steps // 2, 5), 5)
                other["aff_base_384_stage1_model_lists_fp32_as_cluster_numbers"] = {
                    "qk_us": round(per_n[0] * 1e3, 1), "av_us": round(per_n[1] * 1e3, 1)}
                del dn, cn, pn
            if dt == torch.bfloat16:
                # local attention of one block of that stage under mixed precision: one kernel (clusters of 24 as
                # three runs of 8) against what the model ran before it existed - QK on the 144-slot lists, the
                # softmax kernel (fp32 probabilities), the cast of v that clusten/clusten.py:52-53 makes, AV in fp32
                d384 = c384.to("cuda")
                g2 = torch.Generator().manual_seed(1031)
                table384 = torch.randn(rows384, 4, generator=g2).to(dt).cuda()
                pe384 = pe384.cuda()
                bk384, bv384 = torch.randn(128, generator=g2).cuda(), torch.randn(128, generator=g2).cuda()
                cidx24 = (d384.nbhd_idx[:, :, ::24] // 24).to(torch.int32).contiguous()
                plan384 = _native.cluster_attention_plan(cidx24, pe384, None)

                def three_kernels_384():
                    a = _native.qk_forward(d384.query, d384.key, d384.nbhd_idx)
                    p, pb = _native.attn_softmax(a, table384, pe384, None, query=d384.query, blank_key=bk384)
                    return _native.av_forward(p, d384.value.float(), d384.nbhd_idx)

                _, per_x, _, _ = _time_kernels(
                    [lambda: _native.cluster_attention(d384.query, d384.key, d384.value, cidx24, table384, pe384, None,
                                                       bk384, bv384),
                     three_kernels_384,
                     lambda: _native.cluster_attention(d384.query, d384.key, d384.value, None, table384, None, None,
                                                       bk384, bv384, plan=plan384)], max(args.steps // 2, 5), 5)
                fb = 4 * d384.query.numel() * 2 + cidx24.numel() * 4 + pe384.numel() * 8
                other["aff_base_384_stage1_local_attention_bf16_model_lists"] = {
                    "one_kernel_us": round(per_x[0] * 1e3, 1), "three_kernels_us": round(per_x[1] * 1e3, 1),
                    "one_kernel_with_plan_us": round(per_x[2] * 1e3, 1), "one_kernel_algorithmic_bytes": fb,
                    "one_kernel_GBps": round(fb / per_x[0] / 1e6, 1)}
                del d384, table384, pe384, cidx24, plan384
            if dt == torch.float32:
                # merge lists of the same stage: the 144-slot lists of every fourth token, 9216 -> 2304 tokens, C = 128
                w384 = wl.wf_case("aff_base_384_wf", 32, B=16, N=9216, C=128, M=144)
                w384.nbhd_idx = c384.nbhd_idx[:, ::4].contiguous()
                other["aff_base_384_stage1_wf_fp32_model_lists"] = _bench_wf(w384, max(args.steps // 2, 5), 5)
                other["aff_base_384_stage1_backward_fp32_model_lists"] = _bench_backward(c384, w384, 5, 2)
                del w384
        del c384
        other["cfg2_s1_backward_fp32"] = _bench_backward(acase, wcase, max(args.steps // 5, 5), 3)
        other["cfg2_s1_backward_fp32_model_built_lists"] = _bench_backward(
            wl.attn_case("model", 29, B=B, H=2, N=3136, C=32, lists="model_built"), wcase, max(args.steps // 5, 5), 3)
        out["other_configs"] = other
    if not args.no_e2e:
        try:
            out["aff_tiny_224"] = _aff_tiny_throughput(tune_gemms=not (args.no_gemm_tuning or args.quick))
        except Exception as exc:  # noqa: BLE001 - a secondary figure must not cost the line its headline
            out["aff_tiny_224"] = {"error": "%s: %s" % (type(exc).__name__, exc)}
    if not args.no_cpu:
        out["cpu_baseline"] = _cpu_baseline(acase, wcase, total_bytes, B)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()

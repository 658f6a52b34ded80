#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

A step is one forward pass of the fused int8 pipeline over one batch that is already resident in
HBM (fp32 NCHW input -> fp32 logits), replayed from a HIP graph.  Default workload: ResNet-50 v1.5,
batch 64, 3x224x224 N(0,1) inputs, per-channel int8 weights / per-tensor int8 activations,
random-init seeded weights N(0,0.05) with batch norm folded.

Prints ONE JSON line: images/s, plus
  roofline      achieved algorithmic GB/s of the dominant kernel family (the int8 implicit-GEMM
                convolutions) against the 8 TB/s HBM peak, from HIP-event timings of every launch;
  cpu_baseline  the CPU oracle (a port of the reference's formulas) on a bounded sample of the
                same batch, on the host cores of this box;
  extras        int8 GEMM TOPS on the standalone-linear shapes and quantize-kernel GB/s.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
INT8_PEAK_TOPS = 5000.0
# HBM bytes moved by the igemm launches of one ResNet-50 bs64 step, from two rocprofv3 --pmc runs
# (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, factors from a 1 GiB copy in the same runs), keyed by
# (workload, batch, parts the batch is split into): 2.133e9 read + 1.673e9 written with two parts,
# 1.940e9 + 1.666e9 with the batch undivided.  Valid for the default workload only.
MEASURED_TRAFFIC_BYTES = {("resnet50", 64, 2): 3.806e9, ("resnet50", 64, 1): 3.606e9}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="resnet50", choices=["resnet50", "resnet18", "mobilenet_v2", "darknet53_yolov3"])
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--seq-passes", type=int, default=10, help="eager passes timed launch by launch for the roofline")
    ap.add_argument("--calib-images", type=int, default=8)
    ap.add_argument("--cpu-images", type=int, default=0, help="images of the batch the CPU baseline runs (0: the whole batch)")
    ap.add_argument("--fractional-scale", action="store_true",
                    help="quantize with position and fractional scale (steps of absmax/qmax) instead of power-of-two steps")
    ap.add_argument("--streams", type=int, default=2,
                    help="parts the batch is split into inside the HIP graph, each on a stream of its own (1: one launch sequence)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--layers", action="store_true", help="print the per-layer table to stderr")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain 1 GiB device copy (reference dispatch for scaling rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    return ap.parse_args()


def event_time(fn, iters, warm=3):
    """average seconds per call, HIP events on the current stream (the one the kernels run on)"""
    import torch
    for _ in range(warm):
        fn()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    e.synchronize()
    return s.elapsed_time(e) * 1e-3 / iters


def layer_profile(fused, x, iters=20):
    """Time every kernel launch of one forward pass separately (HIP events, `iters` back-to-back
    launches each) and attach the algorithmic bytes / ops of each conv / fc launch."""
    import torch
    ops = torch.ops.torch_mlu
    rows = []
    trace = {}
    fused.forward(x, trace=trace)  # materialise every layer's quantized input once
    torch.cuda.synchronize()
    for l in fused.layers:
        if l.kind not in ("conv", "fc") or l.name in fused._fused_away:
            continue
        lq = fused.q[l.name]
        qx = trace[l.name].get("qx_dev", trace[l.name]["qx"])  # the tensor the kernel reads
        qd = fused.q_demand[l.name][0] if fused.q_demand[l.name] else None
        want_y = fused.f_demand[l.name] or qd is None
        y_half = fused.out_half and l.name in fused.outputs
        ds = fused.shortcut_of.get(l.name) if l.kind == "conv" else None
        extra_macs = extra_bytes = 0
        if ds is not None:  # the block's projection shortcut runs inside this launch
            dq = fused.q[ds.name]
            sx = trace[ds.name]["qx"]
            resid = None
            n_pix = trace[l.name]["y"].numel() // trace[l.name]["y"].shape[-1]
            extra_macs = trace[l.name]["y"].numel() * dq.qw.shape[-1]
            extra_bytes = n_pix * sx.shape[-1] * sx.element_size() + dq.qw.numel() * dq.qw.element_size()

            def run(l=l, lq=lq, qx=qx, qd=qd, want_y=want_y, ds=ds, dq=dq, sx=sx):
                return ops.qconv2d_shortcut(qx, lq.qw, lq.exp2, lq.chan_div, lq.bias, sx, dq.qw, ds.stride, dq.exp2,
                                            dq.chan_div, dq.bias, fused.padding(l), [l.stride, l.stride], [1, 1],
                                            {"none": 0, "relu": 1, "relu6": 2, "leaky": 3}[l.act], want_y, y_half,
                                            qd[0] if qd else 0, qd[1] if qd else 0, 1.0, 0.1, bool(l.add_after))
            route = "mfma+sc"
        elif l.kind == "conv":
            resid = torch.zeros_like(trace[l.name]["y"]) if l.add else None

            def run(l=l, lq=lq, qx=qx, qd=qd, want_y=want_y, resid=resid):
                return ops.qconv2d(qx, lq.qw, lq.exp2, lq.chan_div, lq.bias, resid, fused.padding(l),
                                   [l.stride, l.stride], [1, 1], lq.groups,
                                   {"none": 0, "relu": 1, "relu6": 2, "leaky": 3}[l.act],
                                   want_y, y_half, False, qd[0] if qd else 0, qd[1] if qd else 0, 1.0, 0.1,
                                   bool(l.add_after))
            route = ops.conv2d_route(lq.bw_x, lq.bw_w, list(qx.shape), list(lq.qw.shape[:3]) + [lq.qw.shape[3]],
                                     fused.padding(l), [l.stride, l.stride], [1, 1], lq.groups)
        else:
            def run(lq=lq, qx=qx):
                return ops.qlinear(qx, lq.qw, lq.exp2, lq.chan_div, lq.bias, 0, True, False, False, 0, 0, 1.0)
            resid = None
            route = "gemm"
        y = trace[l.name]["y"]
        n_out = y.numel()
        macs = n_out * (lq.qw.numel() // lq.qw.shape[0]) + extra_macs
        bytes_alg = qx.numel() * qx.element_size() + lq.qw.numel() * lq.qw.element_size() + extra_bytes
        bytes_alg += ((2 if y_half else 4) * n_out if want_y else 0) + (n_out * (qd[0] // 8) if qd else 0) + (4 * n_out if resid is not None else 0)
        t = event_time(run, iters)
        rows.append(dict(name=l.name, route=route, t=t, ops=2 * macs, bytes=bytes_alg))
    return rows


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (every box has one GPU, "
              "the path shards by batch with no communication)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    torch.set_grad_enabled(False)
    import catch_amd  # noqa: F401  (fails loudly if the HIP extension is missing)
    from catch_amd import nets, pipeline

    if args.copy_probe:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")  # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    batch = args.batch or {"resnet50": 64, "resnet18": 64, "mobilenet_v2": 128, "darknet53_yolov3": 16}[args.workload]
    layers = nets.NETS[args.workload]()
    detector = args.workload == "darknet53_yolov3"
    side = 416 if detector else 224
    gen = torch.Generator().manual_seed(1)
    t0 = time.time()
    if detector:
        # int16 activations x int8 weights, q-params in the [bitwidths],[positions] encoding, fp16 outputs
        net = nets.FloatNet(layers, seed=0, weight_std="he").eval()
        x = torch.rand(batch, 3, side, side, generator=gen)
        sd = pipeline.to_position_encoding(pipeline.calibrate(net, x[:min(args.calib_images, 2)], "int16", False), 16, 8)
        what = "int16 activations x int8 weights (per-tensor positions), batch %d, 3x416x416 U(0,1), fp16 outputs" % batch
    else:
        net = nets.FloatNet(layers, seed=0).eval()
        x = torch.randn(batch, 3, side, side, generator=gen)
        sd = pipeline.calibrate(net, x[:args.calib_images], "int8", True)
        what = "int8 (per-channel W, per-tensor act), batch %d, 3x224x224 N(0,1)" % batch
    t_cal = time.time() - t0
    if args.fractional_scale:
        if detector:
            sys.exit("--fractional-scale needs a checkpoint of scales; the detector's holds bit widths and positions")
        what += ", position + fractional scale"
    fused = pipeline.FusedNet(layers, sd, out_half=detector, fractional_scale=args.fractional_scale)
    xg = x.cuda()
    if args.streams < 1:
        sys.exit("--streams must be at least 1")
    while batch % args.streams:  # the largest number of equal parts not above what was asked for
        args.streams -= 1
    static_in, replay = fused.capture(xg, streams=args.streams)
    static_in.copy_(xg)
    for _ in range(args.warmup):
        replay()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(args.steps):
        out = replay()
    e.record()
    torch.cuda.synchronize()
    ms_per_step = s.elapsed_time(e) / args.steps
    value = batch / (ms_per_step * 1e-3)
    outs = out if isinstance(out, tuple) else (out,)
    for o in outs:
        assert torch.isfinite(o.float()).all()

    # ---- per-kernel roofline of the dominant family: the implicit-GEMM convolutions ------------
    # The launches measured are the ones the graph holds: with the batch in `streams` parts, every layer is
    # launched once per part, on that part's images.
    parts = list(xg.chunk(args.streams))
    from catch_amd import _native
    _native.kernel_lib().catchq_set_launch_sharing(args.streams)  # the tile shapes the graph's launches were given
    rows = layer_profile(fused, parts[0])
    # Launch durations in their real sequence: HIP events around every conv/fc launch of eager forward
    # passes on the stream the kernels run on (no graph: a captured launch cannot be bracketed; one part
    # after the other, so without the overlap between the parts' streams that the graph has).  Unlike the
    # back-to-back repetitions of layer_profile these see the caches the way a whole pass leaves them.
    timers = {}
    for i in range(2 + args.seq_passes):
        t_ = timers if i >= 2 else None
        for part in parts:
            fused.forward(part, timers=t_)
    torch.cuda.synchronize()
    _native.kernel_lib().catchq_set_launch_sharing(1)
    # The part of a bracketed duration that is the bracket's, not the kernel's: a pair of events around one small
    # kernel reads T1, around two of them T2; T2 - T1 is one kernel (and the gap before it), so 2*T1 - T2 is what
    # does not grow with the kernels in between.  (An empty pair reads more, 5.1 us: the markers' own processing
    # partly hides behind a kernel when there is one.)
    probe = torch.zeros(1 << 20, device="cuda")

    def bracket(n_kernels, reps=200):
        evs = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(n_kernels):
                probe.add_(1.0)
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) for a, b in evs)[reps // 2] * 1e-3
    bracket(1, 20)
    t1, t2 = bracket(1), bracket(2)
    empty_s = min(max(2 * t1 - t2, 0.0), t1)
    seq = {}
    for name, evs in timers.items():
        pairs = [(evs[i], evs[i + 1]) for i in range(0, len(evs), 2)]
        seq[name] = max(sum(a.elapsed_time(b) for a, b in pairs) / len(pairs) * 1e-3 - empty_s, 1e-7)
    for r in rows:
        r["t_seq"] = seq[r["name"]]
    conv_rows = [r for r in rows if r["route"].startswith("mfma")]
    n_parts = len(parts)  # per step: every row's launch once per part
    t_conv = n_parts * sum(r["t_seq"] for r in conv_rows)
    t_conv_hot = n_parts * sum(r["t"] for r in conv_rows)
    b_conv = n_parts * sum(r["bytes"] for r in conv_rows)
    o_conv = n_parts * sum(r["ops"] for r in conv_rows)
    t_all = n_parts * sum(r["t"] for r in rows)
    if args.layers:
        for r in rows:
            print("%-12s %-9s %8.1f us %7.1f GB/s %7.1f TOPS   in sequence %8.1f us" % (
                r["name"], r["route"], r["t"] * 1e6, r["bytes"] / r["t"] / 1e9, r["ops"] / r["t"] / 1e12,
                r["t_seq"] * 1e6), file=sys.stderr)
        print("sum of conv/fc launches (%d parts of %d images): %.1f us repeated back to back, %.1f us in sequence; graph step: %.1f us" % (
            n_parts, parts[0].shape[0], t_all * 1e6, n_parts * sum(r["t_seq"] for r in rows) * 1e6, ms_per_step * 1e3), file=sys.stderr)
    roofline = {"bound": "hbm", "kernel": "%s (all %d launches of one step: %d layers x %d parts of the batch)" % (
                    "igemm_a16_dma_kernel" if detector else "igemm_i8_dma_kernel + igemm_i8_dual_kernel",
                    n_parts * len(conv_rows), len(conv_rows), n_parts),
                "achieved": round(b_conv / t_conv / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(b_conv / t_conv / 1e9 / HBM_PEAK_GBS, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get((args.workload, batch, n_parts)),
                "avg_launch_us": round(t_conv / max(n_parts * len(conv_rows), 1) * 1e6, 2),
                "timing": "HIP events around each launch of eager forward passes over the parts, in sequence (%d passes), "
                          "minus the bracket's own share, 2*T(pair around one small kernel) - T(pair around two), "
                          "measured in the same run (%.2f us)" % (args.seq_passes, empty_s * 1e6),
                "event_pair_overhead_us": round(empty_s * 1e6, 2),
                "achieved_repeated_launches": round(b_conv / t_conv_hot / 1e9, 1),
                "algorithmic_bytes_per_step": b_conv, "int8_tops": round(o_conv / t_conv / 1e12, 1),
                "mfma_frac": round(o_conv / t_conv / 1e12 / INT8_PEAK_TOPS, 4),
                # the parts' launches overlap in the timed graph, so the step is shorter than the sum of its
                # launches timed one by one; the same bytes over the whole timed step (which also holds the
                # input quantizer and the pooling kernels) bound the family's aggregate rate from below
                "over_timed_region": {"sum_of_launches_us": round(t_conv * 1e6, 1), "graph_step_us": round(ms_per_step * 1e3, 1),
                                      "achieved": round(b_conv / (ms_per_step * 1e-3) / 1e9, 1),
                                      "frac": round(b_conv / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                      "int8_tops": round(o_conv / (ms_per_step * 1e-3) / 1e12, 1)}}

    result = {"metric": "int8 ResNet-50 images/sec bs64 + int8 GEMM TOPS (% MFMA peak), 1 GPU" if args.workload == "resnet50"
              else "int8 %s images/sec" % args.workload,
              "value": round(value, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
              "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
              "dtype": "int16xint8" if detector else "int8", "data": "synthetic",
              "config": {"workload": "%s %s, fused requant pipeline replayed from a HIP graph%s" % (
                  args.workload, what, "" if args.streams <= 1 else " (the batch in %d parts on parallel streams)" % args.streams),
                         "global_batch": batch, "calibration_images": args.calib_images, "graph_streams": args.streams,
                         "gop_per_step": round(2 * nets.conv_macs(layers, batch, side, side) / 1e9, 1)},
              "roofline": roofline}

    if not args.no_extras:
        result["extras"] = extras()
        if args.workload == "resnet50" and not args.fractional_scale:  # the modules quantize in power-of-two steps
            result["extras"]["dropin_modules"] = dropin_flow(net, x, args.calib_images, out)
    if not args.no_cpu_baseline:
        n_cpu = args.cpu_images or batch
        result["cpu_baseline"] = cpu_baseline(layers, sd, x[:n_cpu], outs[0][:n_cpu].float().cpu(),
                                              fused.outputs[0], args.fractional_scale)
        # for context: what the reference's modules do with CPU tensors -- the float network (conv.py:175-177)
        import torch as _t
        t0 = time.time()
        net(x[:n_cpu])
        result["cpu_baseline"]["float_torch_cpu"] = {"value": round(n_cpu / (time.time() - t0), 2), "unit": "images/s",
                                                     "threads": _t.get_num_threads(),
                                                     "what": "the same network in fp32 through PyTorch's CPU kernels"}
    result["calibration_s"] = round(t_cal, 2)
    print(json.dumps(result))


def extras():
    """standalone kernels: int8 linear (config shapes) and quantize streaming rate"""
    import ctypes
    import torch
    ops = torch.ops.torch_mlu
    out = {}
    from catch_amd.pipeline import pos_from_scale

    def gaussian_operands(m, n, k):
        """X[m,k], W[n,k] ~ N(0,1) (seeds 2, 3), X per-tensor int8, W per-channel int8: the standalone linear config"""
        x = torch.randn(m, k, generator=torch.Generator().manual_seed(2)).cuda()
        w = torch.randn(n, k, generator=torch.Generator().manual_seed(3)).cuda()
        pos_x = pos_from_scale(8, 127.0 / x.abs().max().item())
        qx = ops.quantize(x, 8, pos_x, 1.0)
        scales = (127.0 / w.abs().amax(1)).float()
        qw, new_pos, new_scale = ops.quantize_per_channel(w, scales, 8)
        return qx, qw, pos_x + int(new_pos.item()), new_scale

    def time_gemm(a, b, exp2, div, bias, iters):
        return event_time(lambda: ops.qlinear(a, b, exp2, div, bias, 1, True, True, False, 0, 0, 1.0), iters, max(iters // 10, 3))

    for (m, n, k) in ((4096, 3072, 768), (4096, 768, 3072)):
        bias = torch.randn(n, generator=torch.Generator().manual_seed(4)).cuda()
        a, b, exp2, div = gaussian_operands(m, n, k)
        t = time_gemm(a, b, exp2, div, bias, 200)
        out["linear_%dx%dx%d" % (m, n, k)] = {"us": round(t * 1e6, 2), "tops": round(2 * m * n * k / t / 1e12, 1),
                                             "mfma_frac": round(2 * m * n * k / t / 1e12 / INT8_PEAK_TOPS, 4),
                                             "operands": "N(0,1) quantized: X per tensor, W per channel",
                                             "epilogue": "per-channel dequant + bias + ReLU, fp16 out"}
    # a GEMM large enough to be bound by the matrix cores, on two kinds of data: the rate depends on how many
    # operand bits toggle (the chip lowers its clock under high-toggle matrix work)
    m = n = k = 8192
    bias = torch.randn(n, device="cuda")
    a, b, exp2, div = gaussian_operands(m, n, k)
    t_g = time_gemm(a, b, exp2, div, bias, 10)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda")
    b = torch.randint(-128, 128, (n, k), dtype=torch.int8, device="cuda")
    t_u = time_gemm(a, b, -10, div, bias, 10)
    out["gemm_8192x8192x8192"] = {"us_gaussian_operands": round(t_g * 1e6, 1), "tops_gaussian_operands": round(2 * m * n * k / t_g / 1e12, 1),
                                  "us_uniform_operands": round(t_u * 1e6, 1), "tops_uniform_operands": round(2 * m * n * k / t_u / 1e12, 1),
                                  "mfma_frac": round(2 * m * n * k / t_g / 1e12 / INT8_PEAK_TOPS, 4)}
    del a, b
    n = 64 * 256 * 56 * 56  # one ResNet-50 stage-1 activation, 822 MB of fp32: larger than the 256 MB cache
    x = torch.randn(n, device="cuda")
    t = event_time(lambda: ops.quantize(x, 8, -5, 1.0), 20, 3)
    out["quantize_f32_to_i8"] = {"elements": n, "us": round(t * 1e6, 1), "gbs": round(5 * n / t / 1e9, 1),
                                 "hbm_frac": round(5 * n / t / 1e9 / HBM_PEAK_GBS, 4)}
    return out


def dropin_flow(net, x, calib_images, fused_logits):
    """the same network and batch through the module-swap flow of the reference (quantize_dynamic_mlu, one
    torch_mlu::conv2d / linear call per layer, fp32 tensors and ATen ReLU / add / pooling between them)"""
    import torch
    from catch_amd.core.mlu_quantize import quantize_dynamic_mlu
    spec = {"use_avg": False, "data_scale": 1.0, "per_channel": True, "firstconv": False}
    calib = quantize_dynamic_mlu(net, spec, dtype="int8", gen_quant=True)
    calib(x[:calib_images])
    q = quantize_dynamic_mlu(net)
    q.load_state_dict(calib.state_dict())
    q = q.to("cuda")
    xg = x.cuda()
    t = event_time(lambda: q(xg), 10, 3)
    y = q(xg)
    return {"ms_per_step": round(t * 1e3, 3), "images_per_s": round(x.shape[0] / t, 1),
            "logits_equal_fused": bool(torch.equal(y, fused_logits))}


def cpu_baseline(layers, sd, x_sample, gpu_logits, out_name, fractional_scale=False):
    """the oracle's unfused execution of the same network on a few images of the same batch"""
    import numpy as np
    import oracle as orc
    from oracle import netref
    sdn = {k: v.detach().cpu().numpy() for k, v in sd.items()}
    t0 = time.time()
    t, _ = netref.run(layers, sdn, x_sample.numpy(), record=False, fractional_scale=fractional_scale)
    dt = time.time() - t0
    if gpu_logits.dim() == 4:  # logical NCHW -> the oracle's NHWC
        gpu_logits = gpu_logits.permute(0, 2, 3, 1).contiguous()
    want = t[out_name].reshape(gpu_logits.shape)
    span = float(want.max() - want.min())
    err = float(np.abs(want - gpu_logits.numpy()).max())
    return {"value": round(x_sample.shape[0] / dt, 3), "unit": "images/s", "cores": orc.num_threads(), "kind": "port",
            "sample": "%d images of the same batch through the whole network (oracle, OpenMP)" % x_sample.shape[0],
            "gpu_vs_oracle_max_abs": err, "output_range": span, "within_1e-3_of_range": bool(err <= 1e-3 * span)}


if __name__ == "__main__":
    main()

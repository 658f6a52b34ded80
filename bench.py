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
# Where the HBM traffic of the convolution launches was measured (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# `bench.py --graph-only`); the bench line itself reports no traffic figure: it cannot read a counter.
TRAFFIC_PROFILE = {"resnet50": "profiles/igemm_i8_resnet50_bs64_hbm_traffic.md"}
# rocprofv3 --kernel-trace --stats summaries of `bench.py --graph-only`, by (workload, parts of the batch)
KERNEL_PROFILE = {("resnet50", 2): "profiles/resnet50_bs64_graph_two_streams_kernel_stats.md",
                  ("resnet50", 1): "profiles/resnet50_bs64_graph_one_stream_kernel_stats.md",
                  ("mobilenet_v2", 2): "profiles/mobilenet_v2_bs128_kernel_stats.md",
                  ("darknet53_yolov3", 2): "profiles/darknet53_yolov3_bs16_kernel_stats.md"}


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
    ap.add_argument("--chain-links", type=int, default=-1,
                    help="longest residual chain recomputed inside a block's last launch (0: none, -1: the plan's own rule)")
    ap.add_argument("--fuse-blocks", action="store_true",
                    help="inverted-residual blocks as one launch each where the kernel serves the shape (A/B runs)")
    ap.add_argument("--no-fuse-first", action="store_true",
                    help="input quantizer, first convolution and max pooling as three launches (A/B runs)")
    ap.add_argument("--no-fuse-avgpool", action="store_true",
                    help="the last 1x1 convolution and the global average pooling as two launches (A/B runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--layers", action="store_true", help="print the per-layer table to stderr")
    ap.add_argument("--graph-only", action="store_true",
                    help="time the graph replays and launch nothing else (no per-launch passes, no extras, no CPU "
                         "baseline): the mode to run under rocprofv3, whose kernel table then holds the timed region only")
    ap.add_argument("--probe", default="",
                    help="launch one kernel --probe-iters times and exit (for rocprofv3 counter runs): "
                         "gemm:MxNxK (config-2 epilogue), quantize, dequantize, absmax, frame, layer:NAME (that layer's "
                         "launch of the workload), copy, mfma (what the int8 matrix cores sustain: prints its own rates)")
    ap.add_argument("--probe-iters", type=int, default=20)
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


def layer_profile(fused, x, iters=20, only=None):
    """Time every kernel launch of one forward pass separately (HIP events, `iters` back-to-back
    launches each) and attach the algorithmic bytes / ops of each conv / fc launch."""
    import torch
    ops = torch.ops.torch_mlu
    rows = []
    trace = {}
    fused.forward(x, trace=trace)  # materialise every layer's quantized input once
    torch.cuda.synchronize()
    fused_heads = set(h.name for h in fused.head_of.values()
                      if fused.head_fuses(h, *trace[h.name]["qx"].shape[:3]))
    fused_inner = set()  # expansion and depthwise layers that run inside their block's projection launch
    for pname, (bx, bd) in fused.block_of.items():
        if fused.block_fuses(next(l for l in fused.layers if l.name == pname), *trace[bx.name]["qx"].shape[:3]):
            fused_inner.update((bx.name, bd.name))
    first = fused.first_layers_fuse(*x.shape)  # quantizer, first convolution and pooling in one launch
    for l in fused.layers:
        if l.kind not in ("conv", "fc") or l.name in fused._fused_away or l.name in fused_heads or l.name in fused_inner \
                or (only and l.name != only):
            continue
        if first and l is fused.layers[0]:
            lq, pool, d = fused.q[l.name], fused.first_pool, fused.q_demand["input"][0]
            qd = fused.q_demand[pool.name][0]
            code = {"relu": 1, "relu6": 2}[l.act]

            def run(l=l, lq=lq, pool=pool, d=d, qd=qd, code=code):
                return ops.qconv2d_first_layers(x, d[1], d[2], lq.qw, lq.exp2, lq.chan_div, lq.bias, code, qd[1], l.k, l.stride,
                                                l.pad, pool.k, pool.stride, pool.pad)
            pooled = run()
            macs = trace[l.name]["y"].numel() * (lq.qw.numel() // lq.qw.shape[0])
            t = event_time(run, iters)
            rows.append(dict(name=l.name, route="mfma+first", t=t, ops=2 * macs,
                             bytes=x.numel() * 4 + lq.qw.numel() + pooled.numel()))
            continue
        lq = fused.q[l.name]
        qx = trace[l.name].get("qx_dev", trace[l.name]["qx"])  # the tensor the kernel reads
        qd = fused.q_demand[l.name][0] if fused.q_demand[l.name] else None
        want_y = fused.f_demand[l.name] or qd is None
        y_half = fused.out_half and l.name in fused.outputs
        ds = fused.shortcut_of.get(l.name) if l.kind == "conv" else None
        chain = fused.chain_of.get(l.name) if l.kind == "conv" else None
        extra_macs = extra_bytes = 0
        head = fused.head_of.get(l.name) if l.kind == "conv" else None
        block = fused.block_of.get(l.name) if l.kind == "conv" else None
        gap = next((g for g in fused.layers if fused.pooled_conv.get(g.name) is l), None)
        if gap is not None and fused.avgpool_fuses(gap, *qx.shape[:3]):
            # the convolution runs inside the launch of the global average pooling behind it: its fp32 output is never
            # stored, the launch writes the pooled values only
            qds = fused.q_demand[gap.name]
            want_mean = fused.f_demand[gap.name] or len(qds) != 1
            gd = qds[0] if qds else None
            resid = torch.zeros_like(trace[l.name]["y"]) if l.add else None
            code = {"none": 0, "relu": 1, "relu6": 2}[l.act]

            def run(lq=lq, qx=qx, resid=resid, code=code, want_mean=want_mean, gd=gd):
                return ops.qconv2d_avgpool(qx, lq.qw, lq.exp2, lq.chan_div, lq.bias, resid, code, want_mean,
                                           gd[0] if gd else 0, gd[1] if gd else 0, gd[2] if gd else 1.0)
            y = trace[l.name]["y"]
            pooled = y.shape[0] * y.shape[-1]
            t = event_time(run, iters)
            rows.append(dict(name=l.name, route="mfma+avgpool", t=t, ops=2 * y.numel() * (lq.qw.numel() // lq.qw.shape[0]),
                             bytes=qx.numel() + lq.qw.numel() + (4 * y.numel() if resid is not None else 0)
                             + pooled * ((4 if want_mean else 0) + (gd[0] // 8 if gd else 0))))
            continue
        if block is not None and block[0].name in fused_inner:
            # expansion and depthwise layer run inside this launch: the block input and all three filter sets are read,
            # neither hidden tensor is stored
            bx, bd = block
            xq, dq = fused.q[bx.name], fused.q[bd.name]
            hx = trace[bx.name]["qx"]
            resid = torch.zeros_like(trace[l.name]["y"]) if l.add else None
            extra_macs = trace[bx.name]["y"].numel() * xq.qw.shape[-1] + trace[bd.name]["y"].numel() * 9
            extra_bytes = hx.numel() + xq.qw.numel() + dq.qw.numel() - qx.numel()
            code = {"none": 0, "relu": 1, "relu6": 2, "leaky": 3}

            def run(l=l, lq=lq, xq=xq, dq=dq, hx=hx, bx=bx, bd=bd, qd=qd, want_y=want_y, resid=resid):
                return ops.qconv2d_irb(hx, xq.qw, xq.exp2, xq.chan_div, xq.bias, code[bx.act], dq.pos_x, dq.qw, bd.stride,
                                       dq.exp2, dq.chan_div, dq.bias, code[bd.act], lq.pos_x, lq.qw, lq.exp2, lq.chan_div,
                                       lq.bias, resid, want_y, y_half, qd[0] if qd else 0, qd[1] if qd else 0, 1.0)
            route = "mfma+block"
        elif head is not None and head.name in fused_heads:
            # the 1x1 layer in front runs inside this launch: its input and filters are read, its output never stored
            hq = fused.q[head.name]
            hx = trace[head.name]["qx"]
            resid = None
            extra_macs = trace[head.name]["y"].numel() * hq.qw.shape[-1]
            extra_bytes = hx.numel() + hq.qw.numel() - qx.numel()  # instead of this layer's own input tensor

            def run(l=l, lq=lq, hq=hq, hx=hx, qd=qd, want_y=want_y):
                return ops.qconv2d_head(hx, hq.qw, hq.exp2, hq.chan_div, hq.bias, lq.pos_x, lq.qw, lq.exp2, lq.chan_div,
                                        lq.bias, fused.padding(l), [1, 1], [1, 1],
                                        {"none": 0, "relu": 1, "relu6": 2, "leaky": 3}[l.act], want_y, y_half,
                                        qd[0] if qd else 0, qd[1] if qd else 0, 1.0, 0.1)
            route = "mfma+head"
        elif chain is not None:  # the residual chain back to the stage's shortcut is recomputed inside this launch
            resid = None
            n_pix = trace[l.name]["y"].numel() // trace[l.name]["y"].shape[-1]
            cq = [fused.q[c.name] for c in chain]
            xs = [trace[c.name]["qx"] for c in chain]
            for c, k, sx in zip(chain[:-1], cq[:-1], xs[:-1]):
                extra_macs += trace[l.name]["y"].numel() * k.qw.shape[-1]
                extra_bytes += n_pix * sx.shape[-1] * sx.element_size() + k.qw.numel() * k.qw.element_size()

            def run(chain=chain, cq=cq, xs=xs, qd=qd, want_y=want_y):
                return ops.qconv2d_chain(xs, [k.qw for k in cq], [c.stride for c in chain], [k.exp2 for k in cq],
                                         [k.chan_div for k in cq], [k.bias for k in cq], want_y, 8 if qd else 0,
                                         qd[1] if qd else 0)
            route = "mfma+chain%d" % len(chain)
        elif ds is not None:  # the block's projection shortcut runs inside this launch
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


def plan_launches(fused, n, h, w):
    """Every launch of one untraced forward pass over n images of h x w, in launch order, with its algorithmic
    bytes (the tensors the fused plan moves: integer inputs and weights, fp32 residual read, fp32 / fp16 and
    integer outputs written) and integer operations, from the layer shapes alone (nothing is launched)."""
    rows, shape = [], {}
    pooled_inside = set()  # 1x1 convolutions that run inside the launch of the global average pooling behind them
    cin = fused.cdev["input"]
    first = fused.first_layers_fuse(n, fused.chan["input"], h, w)  # quantizer, first convolution and pooling in one launch
    for d in fused.q_demand["input"] if not first else ():
        if fused.stem:
            sp = fused.stem["pad"]
            oh, ow = h + 2 * sp, w + 2 * sp + fused.stem["extra"]
        else:
            oh, ow = h, w
        shape[("input", "q")] = (oh, ow)
        rows.append(dict(name="input", kind="quantize", ops=0, bytes=n * fused.chan["input"] * h * w * 4 + n * oh * ow * cin * d[0] // 8))
    shape["input"] = (h, w)
    for l in fused.layers:
        if l.kind == "conv":
            hi, wi = shape[l.src]
            ho, wo = (hi + 2 * l.pad - l.k) // l.stride + 1, (wi + 2 * l.pad - l.k) // l.stride + 1
            shape[l.name] = (ho, wo)
            if l.name in fused._fused_away or fused.head_fuses(l, n, hi, wi):
                continue
            gap = next((g for g in fused.layers if fused.pooled_conv.get(g.name) is l), None)
            if gap is not None and fused.avgpool_fuses(gap, n, hi, wi):
                lq, qds = fused.q[l.name], fused.q_demand[gap.name]
                n_out = n * ho * wo * fused.cdev[l.name]
                k = lq.qw.numel() // lq.qw.shape[0]
                pooled_bytes = n * fused.cdev[l.name] * ((4 if (fused.f_demand[gap.name] or len(qds) != 1) else 0)
                                                          + (qds[0][0] // 8 if qds else 0))
                rows.append(dict(name=l.name, kind="conv", ops=2 * n_out * k, m=n * ho * wo, n=fused.cdev[l.name], k=k,
                                 bytes=n * hi * wi * fused.cdev[l.src] + lq.qw.numel() + (4 * n_out if l.add else 0) + pooled_bytes))
                pooled_inside.add(l.name)
                continue
            if first and l is fused.layers[0]:
                lq, pool = fused.q[l.name], fused.first_pool
                hp, wp = (ho + 2 * pool.pad - pool.k) // pool.stride + 1, (wo + 2 * pool.pad - pool.k) // pool.stride + 1
                rows.append(dict(name=l.name, kind="conv", ops=2 * n * ho * wo * fused.cdev[l.name] * (lq.qw.numel() // lq.qw.shape[0]),
                                 bytes=n * fused.chan["input"] * h * w * 4 + lq.qw.numel() + n * hp * wp * fused.cdev[l.name],
                                 m=n * ho * wo, n=fused.cdev[l.name], k=lq.qw.numel() // lq.qw.shape[0]))
                continue
            if l.name in fused._block_inner:
                bp = next(m for m in fused.layers if m.name == fused._block_inner[l.name])
                if fused.block_fuses(bp, n, *shape[fused.block_of[bp.name][0].src]):
                    continue
            lq = fused.q[l.name]
            n_out = n * ho * wo * fused.cdev[l.name]
            ih, iw = shape[("input", "q")] if (fused.stem and l.name == fused.stem["name"]) else (hi, wi)
            macs = n_out * (lq.qw.numel() // lq.qw.shape[0])
            b = n * ih * iw * fused.cdev[l.src] * lq.bw_x // 8 + lq.qw.numel() * lq.qw.element_size()
            ds = fused.shortcut_of.get(l.name)
            chain = fused.chain_of.get(l.name)
            k_extra = 0
            head = fused.head_of.get(l.name)
            if head is not None and fused.head_fuses(head, n, hi, wi):
                hq = fused.q[head.name]
                macs += n * hi * wi * fused.cdev[head.name] * hq.qw.shape[-1]
                b += n * hi * wi * (fused.cdev[head.src] - fused.cdev[l.src]) + hq.qw.numel()
            block = fused.block_of.get(l.name)
            if block is not None and fused.block_fuses(l, n, *shape[block[0].src]):
                bx, bd = block
                xq, dq = fused.q[bx.name], fused.q[bd.name]
                bh, bw = shape[bx.src]
                macs += n * bh * bw * fused.cdev[bx.name] * xq.qw.shape[-1] + n * ho * wo * fused.cdev[bd.name] * 9
                b += n * bh * bw * fused.cdev[bx.src] - n * hi * wi * fused.cdev[l.src] + xq.qw.numel() + dq.qw.numel()
            if chain is not None:
                # every earlier link of the residual chain is recomputed inside this launch: its int8 input (the
                # pixels the 1x1 taps touch) and its weights are read, its 2*K operations per output repeated
                for c in chain[:-1]:
                    cq = fused.q[c.name]
                    macs += n_out * cq.qw.shape[-1]
                    k_extra += cq.qw.shape[-1]
                    b += n * ho * wo * fused.cdev[c.src] * cq.bw_x // 8 + cq.qw.numel() * cq.qw.element_size()
            elif ds is not None:
                dq = fused.q[ds.name]
                macs += n_out * dq.qw.shape[-1]
                k_extra = dq.qw.shape[-1]
                b += n * ho * wo * fused.cdev[ds.src] * dq.bw_x // 8 + dq.qw.numel() * dq.qw.element_size()
            elif l.add:
                b += 4 * n_out
            qd = fused.q_demand[l.name][0] if fused.q_demand[l.name] else None
            want_y = fused.f_demand[l.name] or qd is None
            y_half = fused.out_half and l.name in fused.outputs
            b += ((2 if y_half else 4) * n_out if want_y else 0) + (n_out * qd[0] // 8 if qd else 0)
            rows.append(dict(name=l.name, kind="conv", ops=2 * macs, bytes=b, m=n * ho * wo, n=fused.cdev[l.name],
                             k=lq.qw.numel() // lq.qw.shape[0] + k_extra))
            for d in fused.q_demand[l.name][1:]:
                rows.append(dict(name=l.name, kind="quantize", ops=0, bytes=n_out * 4 + n_out * d[0] // 8))
        elif l.kind == "fc":
            lq = fused.q[l.name]
            shape[l.name] = (1, 1)
            k = lq.qw.shape[1]
            rows.append(dict(name=l.name, kind="fc", ops=2 * n * k * lq.qw.shape[0], m=n, n=lq.qw.shape[0], k=k,
                             bytes=n * k * lq.bw_x // 8 + lq.qw.numel() * lq.qw.element_size() + 4 * n * lq.qw.shape[0]))
        elif l.kind == "maxpool":
            hi, wi = shape[l.src]
            ho, wo = (hi + 2 * l.pad - l.k) // l.stride + 1, (wi + 2 * l.pad - l.k) // l.stride + 1
            shape[l.name] = (ho, wo)
            for form in fused._forms(l.name) if not (first and l is fused.first_pool) else ():
                e = 4 if form == ("f",) else form[0] // 8
                rows.append(dict(name=l.name, kind="maxpool", ops=0, bytes=n * fused.cdev[l.src] * e * (hi * wi + ho * wo)))
        elif l.kind == "gap":
            hi, wi = shape[l.src]
            shape[l.name] = (1, 1)
            c = fused.cdev[l.src]
            if l.src in pooled_inside:
                for d in fused.q_demand[l.name][1:]:
                    rows.append(dict(name=l.name, kind="quantize", ops=0, bytes=n * c * (4 + d[0] // 8)))
            elif fused.f_demand[l.name] or not fused.q_demand[l.name]:
                rows.append(dict(name=l.name, kind="avgpool", ops=0, bytes=n * c * 4 * (hi * wi + 1)))
                for d in fused.q_demand[l.name]:
                    rows.append(dict(name=l.name, kind="quantize", ops=0, bytes=n * c * (4 + d[0] // 8)))
            else:
                for d in fused.q_demand[l.name]:
                    rows.append(dict(name=l.name, kind="avgpool+quantize", ops=0, bytes=n * c * (4 * hi * wi + d[0] // 8)))
        elif l.kind == "upsample":
            hi, wi = shape[l.src]
            shape[l.name] = (hi * 2, wi * 2)
            for form in fused._forms(l.name):  # torch's repeat_interleave, twice: rows doubled, then columns
                e = 4 if form == ("f",) else form[0] // 8
                rows.append(dict(name=l.name, kind="upsample", ops=0, bytes=n * fused.cdev[l.src] * e * hi * wi * 3))
                rows.append(dict(name=l.name, kind="upsample", ops=0, bytes=n * fused.cdev[l.src] * e * hi * wi * 6))
        elif l.kind == "concat":
            shape[l.name] = shape[l.src[0]]
            hi, wi = shape[l.name]
            for form in fused._forms(l.name):
                e = 4 if form == ("f",) else form[0] // 8
                rows.append(dict(name=l.name, kind="concat", ops=0, bytes=2 * n * fused.cdev[l.name] * e * hi * wi))
    return rows


def head_hw(fused, head, side):
    """extent of the tensor the 1x1 layer `head` reads, for a network input of side x side"""
    shape = {"input": (side, side)}
    for l in fused.layers:
        if l is head:
            return shape[l.src]
        if l.kind in ("conv", "maxpool"):
            hi, wi = shape[l.src]
            shape[l.name] = ((hi + 2 * l.pad - l.k) // l.stride + 1, (wi + 2 * l.pad - l.k) // l.stride + 1)
        elif l.kind == "upsample":
            shape[l.name] = tuple(2 * v for v in shape[l.src])
        elif l.kind == "concat":
            shape[l.name] = shape[l.src[0]]
        else:
            shape[l.name] = (1, 1)
    raise KeyError(head.name)


def bound_of(ops, nbytes):
    """which roof the launch's algorithmic work sits under: the time its bytes need at the HBM peak against the
    time its operations need at the int8 matrix peak"""
    return "hbm" if nbytes / (HBM_PEAK_GBS * 1e9) >= ops / (INT8_PEAK_TOPS * 1e12) else "mfma"


def run_probe(args):
    """one kernel, launched --probe-iters times on the current stream: what a rocprofv3 --pmc run should see"""
    import torch
    import catch_amd  # noqa: F401
    ops = torch.ops.torch_mlu
    what = args.probe
    it = args.probe_iters
    if what == "copy":  # the reference dispatch for scaling FETCH_SIZE / WRITE_SIZE: 1 GiB read, 1 GiB written
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(it):
            dst.copy_(src)
        desc = "1 GiB fp32 copy"
    elif what.startswith("gemm:"):
        m, n, k = (int(v) for v in what[5:].split("x"))
        a, b, exp2, div, bias = gaussian_linear_operands(m, n, k)
        t = event_time(lambda: ops.qlinear(a, b, exp2, div, bias, 1, True, True, False, 0, 0, 1.0), it, 3)
        desc = "int8 GEMM %dx%dx%d, per-channel dequant + bias + ReLU, fp16 out: %.1f us per launch, %.1f TOPS" % (
            m, n, k, t * 1e6, 2 * m * n * k / t / 1e12)
    elif what == "mfma":
        print(json.dumps({"probe": what, "mfma_ceiling": mfma_ceiling(seconds=2.0)}))
        return
    elif what in ("dequantize", "absmax", "frame"):
        fn, nbytes, desc = streaming_cases()[{"dequantize": "dequantize_i8_to_f32", "absmax": "quantize_param_f32",
                                              "frame": "quantize_frame"}[what]]
        for _ in range(it):
            fn()
    elif what == "quantize":
        n = 64 * 256 * 56 * 56
        xs = [torch.randn(n, device="cuda") for _ in range(6)]
        for i in range(it):
            ops.quantize(xs[i % 6], 8, -5, 1.0)
        desc = "quantize fp32 -> int8, %d elements, 6 rotating inputs" % n
    elif what.startswith("layer:"):
        fused, xg, _ = build_workload(args)
        parts = list(xg.chunk(args.streams))
        ops.set_launch_sharing(args.streams)
        rows = layer_profile(fused, parts[0], iters=it, only=what[6:])
        ops.set_launch_sharing(1)
        desc = "%s of %s, %d images: %.2f us, %.1f GB/s, %.1f TOPS" % (
            what[6:], args.workload, parts[0].shape[0], rows[0]["t"] * 1e6, rows[0]["bytes"] / rows[0]["t"] / 1e9,
            rows[0]["ops"] / rows[0]["t"] / 1e12)
    else:
        sys.exit("unknown --probe " + what)
    torch.cuda.synchronize()
    print(json.dumps({"probe": what, "iters": it, "what": desc}))


def mfma_ceiling(seconds=1.0):
    """The rate a register-resident loop of v_mfma_i32_32x32x32_i8 (no memory access, two waves per SIMD) sustains on
    operands of three kinds; the device lowers its clock under high-toggle matrix work, so the rate depends on them."""
    import ctypes
    import torch
    from catch_amd import _native
    lib = _native.kernel_lib()
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    blocks, iters = 512, 20000
    g = torch.Generator().manual_seed(1234)
    kinds = {"zero_operands": torch.zeros(1 << 20, dtype=torch.int8),
             "uniform_random_bytes": torch.randint(-128, 128, (1 << 20,), generator=g, dtype=torch.int8),
             "normal_bytes_sigma_32": (torch.randn(1 << 20, generator=g) * 32).round().clamp(-128, 127).to(torch.int8)}
    out = {}
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for name, host in kinds.items():
        dev = host.cuda()

        def run(n_it):
            _native.check(lib.catchq_diag_mfma_i8_loop(ctypes.c_void_p(dev.data_ptr()), n_it, blocks,
                                                       ctypes.c_void_p(sink.data_ptr()), stream), "mfma loop")
        run(1000)
        torch.cuda.synchronize()
        total_s = total_ops = 0.0
        while total_s < seconds:
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            run(iters)
            e.record()
            e.synchronize()
            total_s += s.elapsed_time(e) * 1e-3
            total_ops += blocks * 4.0 * iters * 4 * 65536
        out[name] = {"tops": round(total_ops / total_s / 1e12, 1), "frac_of_peak": round(total_ops / total_s / 1e12 / INT8_PEAK_TOPS, 4)}
    return out


def streaming_cases():
    """the streaming kernels beside quantize fp32 -> int8, each over inputs in rotation (6 buffers, so that no launch
    finds its operands in the 256 MB last-level cache): name -> (launch, algorithmic bytes per launch, description)"""
    import torch
    ops = torch.ops.torch_mlu
    n = 64 * 256 * 56 * 56  # one ResNet-50 stage-1 activation: 51.4 M elements
    state = {"i": 0}

    def rot(bufs):
        state["i"] = (state["i"] + 1) % len(bufs)
        return bufs[state["i"]]
    cases = {}
    q8 = [torch.randint(-128, 128, (n,), dtype=torch.int8, device="cuda") for _ in range(6)]
    cases["dequantize_i8_to_f32"] = (lambda: ops.dequantize(rot(q8), -5, 1.7), 5 * n,
                                     "int8 -> fp32, y = q * 2^-5 / 1.7, %d elements" % n)
    x32 = [torch.randn(n, device="cuda") for _ in range(6)]
    cases["quantize_param_f32"] = (lambda: ops.quantize_param(rot(x32), 8, 1), 4 * n,
                                   "max-abs reduction + position and scale, fp32, %d elements (two launches)" % n)
    cases["quantize_f32_to_i16"] = (lambda: ops.quantize(rot(x32), 16, -12, 1.0), 6 * n, "fp32 -> int16, %d elements" % n)
    x16 = [t.half() for t in x32]
    cases["quantize_f16_to_i8"] = (lambda: ops.quantize(rot(x16), 8, -5, 1.0), 3 * n, "fp16 -> int8, %d elements" % n)
    imgs = [torch.randn(64, 3, 224, 224, device="cuda") for _ in range(12)]
    cases["quantize_frame"] = (lambda: ops.quantize_nhwc_frame(rot(imgs), 8, -5, 4, 230, 231, 3, 3, 1.0),
                               64 * 3 * 224 * 224 * 4 + 64 * 230 * 231 * 4,
                               "network input 64x3x224x224 fp32 NCHW -> int8 NHWC (4 channels) inside the first layer's zero "
                               "frame [64,230,231,4]")
    return cases


def gaussian_linear_operands(m, n, k):
    """X[m,k], W[n,k] ~ N(0,1) (seeds 2, 3), bias N(0,1) (seed 4); X per-tensor int8, W per-channel int8:
    the standalone linear configuration.  -> qx, qw, exp2, new_scale, bias"""
    import torch
    from catch_amd.pipeline import pos_from_scale
    ops = torch.ops.torch_mlu
    x = torch.randn(m, k, generator=torch.Generator().manual_seed(2)).cuda()
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(3)).cuda()
    bias = torch.randn(n, generator=torch.Generator().manual_seed(4)).cuda()
    pos_x = pos_from_scale(8, 127.0 / x.abs().max().item())
    qx = ops.quantize(x, 8, pos_x, 1.0)
    scales = (127.0 / w.abs().amax(1)).float()
    qw, new_pos, new_scale = ops.quantize_per_channel(w, scales, 8)
    return qx, qw, pos_x + int(new_pos.item()), new_scale, bias


def build_workload(args):
    """-> (fused plan, input batch on the device, dict(net, x, sd, layers, batch, side, what, detector, t_cal))"""
    import torch
    from catch_amd import nets, pipeline
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
    fused = pipeline.FusedNet(layers, sd, out_half=detector, fractional_scale=args.fractional_scale,
                              chain_links=None if args.chain_links < 0 else args.chain_links,
                              fuse_blocks=getattr(args, "fuse_blocks", False),
                              fuse_first_layers=not getattr(args, "no_fuse_first", False),
                              fuse_avgpool=not getattr(args, "no_fuse_avgpool", False))
    if args.streams < 1:
        sys.exit("--streams must be at least 1")
    while batch % args.streams:  # the largest number of equal parts not above what was asked for
        args.streams -= 1
    return fused, x.cuda(), dict(net=net, x=x, sd=sd, layers=layers, batch=batch, side=side, what=what,
                                 detector=detector, t_cal=t_cal)


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

    if args.probe:
        run_probe(args)
        return
    if args.copy_probe:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")  # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    fused, xg, w_ = build_workload(args)
    net, x, sd, layers, batch, side, what, detector, t_cal = (w_[k] for k in ("net", "x", "sd", "layers", "batch", "side",
                                                                               "what", "detector", "t_cal"))
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

    launches = plan_launches(fused, batch // args.streams, side, side)
    config = {"workload": "%s %s, fused requant pipeline replayed from a HIP graph%s" % (
        args.workload, what, "" if args.streams <= 1 else " (the batch in %d parts on parallel streams)" % args.streams),
              "global_batch": batch, "calibration_images": args.calib_images, "graph_streams": args.streams,
              "gop_per_step": round(2 * nets.conv_macs(layers, batch, side, side) / 1e9, 1),
              # blocks whose residual branch is recomputed from int8 tensors inside their last launch: links per launch
              "residual_chains": {n: len(c) for n, c in fused.chain_of.items()},
              # 3x3 layers whose launch also computes the 1x1 layer in front of them
              "fused_heads": sorted(n for n, h in fused.head_of.items() if fused.head_fuses(h, batch // args.streams, *head_hw(fused, h, side))),
              "fused_blocks": sorted(n for n, (bx, bd) in fused.block_of.items()
                                     if fused.block_fuses(next(l for l in fused.layers if l.name == n), batch // args.streams,
                                                          *head_hw(fused, bx, side))),
              # input quantizer, first convolution and max pooling in one launch
              "fused_first_layers": fused.first_layers_fuse(batch // args.streams, fused.chan["input"], side, side),
              # 1x1 convolutions that run inside the launch of the global average pooling behind them
              "fused_avgpool": sorted(c.name for g, c in fused.pooled_conv.items()
                                      if fused.avgpool_fuses(next(l for l in fused.layers if l.name == g), batch // args.streams,
                                                             *head_hw(fused, c, side)))}
    metric = ("int8 ResNet-50 images/sec bs64 + int8 GEMM TOPS (% MFMA peak), 1 GPU" if args.workload == "resnet50"
              else "int8 %s images/sec" % args.workload)
    if args.graph_only:
        # nothing but the graph replays has been launched since the capture: a kernel trace of this run holds the
        # timed region (plus the capture's own warm-up passes); the launch list names what one part's pass runs
        conv_b = args.streams * sum(r["bytes"] for r in launches if r["kind"] == "conv")
        all_b = args.streams * sum(r["bytes"] for r in launches)
        print(json.dumps({"metric": metric, "value": round(value, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps,
                          "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
                          "scaling": "weak", "vs_baseline": None, "dtype": "int16xint8" if detector else "int8",
                          "data": "synthetic", "config": config,
                          "roofline": {"bound": "hbm", "kernel": "whole timed step (graph replays only)",
                                       "achieved": round(all_b / (ms_per_step * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                                       "unit": "GB/s", "frac": round(all_b / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                       "traffic": None, "algorithmic_bytes_per_step": all_b,
                                       "algorithmic_bytes_of_the_convolutions": conv_b},
                          "launches_per_part": [[r["name"], r["kind"], r["bytes"], r["ops"]] for r in launches]}))
        return

    # ---- per-kernel roofline of the dominant family: the implicit-GEMM convolutions ------------
    # The launches measured are the ones the graph holds: with the batch in `streams` parts, every layer is
    # launched once per part, on that part's images.
    parts = list(xg.chunk(args.streams))
    torch.ops.torch_mlu.set_launch_sharing(args.streams)  # the tile shapes the graph's launches were given
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
    torch.ops.torch_mlu.set_launch_sharing(1)
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
    analytic = {r["name"]: r for r in launches if r["kind"] in ("conv", "fc")}
    for r in rows:
        r["t_seq"] = seq[r["name"]]
        a = analytic[r["name"]]
        assert (a["bytes"], a["ops"]) == (r["bytes"], r["ops"]), "launch accounting differs for %s: %r vs %r" % (r["name"], a, r)
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
                    "igemm_a16_dma_kernel" if detector else "igemm_i8_dma_kernel + conv3x3_halo_kernel + igemm_i8_chain_kernel",
                    n_parts * len(conv_rows), len(conv_rows), n_parts),
                "achieved": round(b_conv / t_conv / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(b_conv / t_conv / 1e9 / HBM_PEAK_GBS, 4),
                "traffic": None, "traffic_profile": TRAFFIC_PROFILE.get(args.workload),
                # the committed kernel trace of the same graph whose per-launch durations give the same fraction
                "frac_profile": KERNEL_PROFILE.get((args.workload, args.streams)),
                "frac_over_timed_step": round(b_conv / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
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

    if fused.chain_of:
        # The residual chains take fp32 traffic out of the plan, so the fractions above divide fewer bytes by a
        # shorter step.  For comparison with a plan that streams every block's fp32 output (what these launches
        # replaced): that plan's algorithmic bytes over the same timed step.
        plain = pipeline.FusedNet(layers, sd, out_half=detector, fractional_scale=args.fractional_scale, chain_links=0)
        b_plain = args.streams * sum(r["bytes"] for r in plan_launches(plain, batch // args.streams, side, side)
                                     if r["kind"] in ("conv", "fc"))
        roofline["over_timed_region"]["bytes_of_the_block_by_block_plan"] = {
            "algorithmic_bytes_per_step": b_plain, "achieved": round(b_plain / (ms_per_step * 1e-3) / 1e9, 1),
            "frac": round(b_plain / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        del plain

    result = {"metric": metric,
              "value": round(value, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
              "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
              "dtype": "int16xint8" if detector else "int8", "data": "synthetic",
              "config": config, "roofline": roofline,
              # every conv / fc launch of one part, timed in sequence: [layer, M, N, K, us, GB/s, TOPS, which roof its
              # algorithmic work sits under, fraction of that roof]
              "layers": [[r["name"], analytic[r["name"]]["m"], analytic[r["name"]]["n"], analytic[r["name"]]["k"],
                          round(r["t_seq"] * 1e6, 1), round(r["bytes"] / r["t_seq"] / 1e9), round(r["ops"] / r["t_seq"] / 1e12),
                          bound_of(r["ops"], r["bytes"]),
                          round(max(r["bytes"] / (HBM_PEAK_GBS * 1e9), r["ops"] / (INT8_PEAK_TOPS * 1e12)) / r["t_seq"], 3)]
                         for r in rows]}

    if not args.no_extras:
        result["extras"] = extras()
        if args.workload == "resnet50":
            result["extras"].update(other_networks())
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
        # one thread of the same oracle on one image, for a per-core figure
        import oracle as orc
        n_thr = orc.num_threads()
        orc.set_num_threads(1)
        one = cpu_baseline(layers, sd, x[:1], outs[0][:1].float().cpu(), fused.outputs[0], args.fractional_scale)
        orc.set_num_threads(n_thr)
        result["cpu_baseline"]["one_thread"] = {"value": one["value"], "unit": "images/s", "cores": 1,
                                                "sample": "1 image of the same batch through the whole network"}
    result["calibration_s"] = round(t_cal, 2)
    print(json.dumps(result))


def extras():
    """standalone kernels: int8 linear (config shapes) and quantize streaming rate"""
    import torch
    ops = torch.ops.torch_mlu
    out = {}

    def alternating(ours, vendor, iters, rounds=7):
        """median seconds per call of each, timed in alternating bursts of `iters` launches behind untimed ones: the
        clock of the device drifts with what it has just been doing, so the two are measured side by side"""
        import statistics
        to, tv = [], []
        try:
            event_time(vendor, iters, 5)
        except Exception as exc:  # the library may refuse a shape
            vendor, tv = None, str(exc)[:80]
        event_time(ours, iters, 5)
        for _ in range(rounds):
            to.append(event_time(ours, iters, 2))
            if vendor is not None:
                tv.append(event_time(vendor, iters, 2))
        return statistics.median(to), (statistics.median(tv) if vendor is not None else tv)

    def gemm_pair(a, b, exp2, div, bias, iters):
        """this library's GEMM with the config-2 epilogue, and the same integer product through torch._int_mm (the
        vendor GEMM library: int32 output, no epilogue -- context from the same box, not a like-for-like launch)"""
        bt = b.t()
        return alternating(lambda: ops.qlinear(a, b, exp2, div, bias, 1, True, True, False, 0, 0, 1.0),
                           lambda: torch._int_mm(a, bt), iters)

    for (m, n, k) in ((4096, 3072, 768), (4096, 768, 3072)):
        a, b, exp2, div, bias = gaussian_linear_operands(m, n, k)
        t, tv = gemm_pair(a, b, exp2, div, bias, 100)
        out["linear_%dx%dx%d" % (m, n, k)] = {"us": round(t * 1e6, 2), "tops": round(2 * m * n * k / t / 1e12, 1),
                                             "mfma_frac": round(2 * m * n * k / t / 1e12 / INT8_PEAK_TOPS, 4),
                                             "operands": "N(0,1) quantized: X per tensor, W per channel",
                                             "epilogue": "per-channel dequant + bias + ReLU, fp16 out",
                                             "torch_int_mm_us": round(tv * 1e6, 2) if isinstance(tv, float) else tv}
    # a GEMM large enough to be bound by the matrix cores, on two kinds of data: the rate depends on how many
    # operand bits toggle (the chip lowers its clock under high-toggle matrix work)
    m = n = k = 8192
    a, b, exp2, div, bias = gaussian_linear_operands(m, n, k)
    t_g, tv_g = gemm_pair(a, b, exp2, div, bias, 10)
    a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda")
    b = torch.randint(-128, 128, (n, k), dtype=torch.int8, device="cuda")
    t_u, tv_u = gemm_pair(a, b, -10, div, bias, 10)
    a.zero_()
    b.zero_()
    t_z = event_time(lambda: ops.qlinear(a, b, -10, div, bias, 1, True, True, False, 0, 0, 1.0), 20, 5)
    out["gemm_8192x8192x8192"] = {"us_gaussian_operands": round(t_g * 1e6, 1), "tops_gaussian_operands": round(2 * m * n * k / t_g / 1e12, 1),
                                  "us_uniform_operands": round(t_u * 1e6, 1), "tops_uniform_operands": round(2 * m * n * k / t_u / 1e12, 1),
                                  "us_zero_operands": round(t_z * 1e6, 1), "tops_zero_operands": round(2 * m * n * k / t_z / 1e12, 1),
                                  "mfma_frac": round(2 * m * n * k / t_g / 1e12 / INT8_PEAK_TOPS, 4),
                                  "timing": "medians of 7 alternating bursts of 10 launches each (this library, then the vendor's)",
                                  "torch_int_mm_us_gaussian": round(tv_g * 1e6, 1) if isinstance(tv_g, float) else tv_g,
                                  "torch_int_mm_us_uniform": round(tv_u * 1e6, 1) if isinstance(tv_u, float) else tv_u}
    del a, b
    # quantize fp32 -> int8: 4 B read + 1 B written per element.  One ResNet-50 stage-1 activation (51.4 M elements)
    # is 206 MB in + 51 MB out, about the size of the 256 MB last-level cache: repeated over one buffer pair that is
    # a warm figure.  The cold one rotates over 6 pairs (1.54 GB), so no launch finds its operands cached.
    n = 64 * 256 * 56 * 56
    xs = [torch.randn(n, device="cuda") for _ in range(6)]
    t_w = event_time(lambda: ops.quantize(xs[0], 8, -5, 1.0), 24, 3)
    state = {"i": 0}

    def cold():
        state["i"] = (state["i"] + 1) % 6
        return ops.quantize(xs[state["i"]], 8, -5, 1.0)
    t_c = event_time(cold, 24, 6)
    out["quantize_f32_to_i8"] = {"elements": n, "us": round(t_c * 1e6, 1), "gbs": round(5 * n / t_c / 1e9, 1),
                                 "hbm_frac": round(5 * n / t_c / 1e9 / HBM_PEAK_GBS, 4),
                                 "working_set": "6 input buffers in rotation, 1.23 GB of fp32 (cold: nothing cached)",
                                 "warm": {"us": round(t_w * 1e6, 1), "gbs": round(5 * n / t_w / 1e9, 1),
                                          "hbm_frac": round(5 * n / t_w / 1e9 / HBM_PEAK_GBS, 4),
                                          "working_set": "one 206 MB input over and over (about the last-level cache's size)"}}
    del xs
    # the other streaming kernels, cold
    for name, (fn, nbytes, desc) in streaming_cases().items():
        t = event_time(fn, 24, 6)
        out[name] = {"us": round(t * 1e6, 1), "gbs": round(nbytes / t / 1e9, 1), "hbm_frac": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4),
                     "what": desc, "working_set": "inputs in rotation (cold: nothing cached)"}
    torch.cuda.empty_cache()
    return out


def other_networks(steps=20):
    """the other two network configurations, each as its own fused plan replayed from a HIP graph (two parts of the
    batch on parallel streams): throughput, algorithmic bytes and integer operations of one step, fractions of the roofs"""
    import argparse as _ap
    import torch
    from catch_amd import nets
    out = {}
    for workload, key in (("mobilenet_v2", "mobilenet_v2_bs128"), ("darknet53_yolov3", "darknet53_yolov3_bs16")):
        a = _ap.Namespace(workload=workload, batch=0, calib_images=8, fractional_scale=False, streams=2, chain_links=-1)
        fused, xg, w_ = build_workload(a)
        static_in, replay = fused.capture(xg, streams=a.streams)
        static_in.copy_(xg)
        for _ in range(5):
            replay()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(steps):
            o = replay()
        e.record()
        torch.cuda.synchronize()
        ms = s.elapsed_time(e) / steps
        for t in (o if isinstance(o, tuple) else (o,)):
            assert torch.isfinite(t.float()).all()
        launches = plan_launches(fused, w_["batch"] // a.streams, w_["side"], w_["side"])
        nbytes = a.streams * sum(r["bytes"] for r in launches)
        nops = 2 * nets.conv_macs(w_["layers"], w_["batch"], w_["side"], w_["side"])
        mfma_ops = nops * (2 if w_["detector"] else 1)  # an int16 x int8 product is two int8 matrix-core passes
        out[key] = {"images_per_s": round(w_["batch"] / (ms * 1e-3), 1), "ms_per_step": round(ms, 4), "steps": steps,
                    "what": w_["what"], "algorithmic_bytes_per_step": nbytes, "gop_per_step": round(nops / 1e9, 1),
                    "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                    "tops": round(nops / (ms * 1e-3) / 1e12, 1),
                    "mfma_frac": round(mfma_ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4)}
        del fused, static_in, replay, xg, w_
        torch.cuda.empty_cache()
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

"""Lowering of traced drop-in models (torch_mlu::conv2d / linear nodes + float neighbours) to the
fused integer plan: the lowered network must reproduce, bit for bit, the plan built directly from
the architecture description and the same checkpoint."""
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    import catch_amd  # noqa: F401
    from catch_amd import jit, nets, pipeline
    from catch_amd.core.mlu_quantize import quantize_dynamic_mlu

torch.set_grad_enabled(False)


def note(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def dropin_model(layers, x, seed, weight_std, per_channel=True):
    net = nets.FloatNet(layers, seed=seed, weight_std=weight_std).eval()
    spec = {"use_avg": False, "data_scale": 1.0, "per_channel": per_channel, "firstconv": False, "iteration": 1}
    calib = quantize_dynamic_mlu(net, spec, dtype="int8", gen_quant=True)
    calib(x)
    qnet = quantize_dynamic_mlu(net)
    qnet.load_state_dict(calib.state_dict())
    return net, qnet.to("cuda").eval()


def test_lowering_with_fractional_scales():
    """the converters' general form (position + fractional scale per tensor / per axis): the lowered plan equals
    the plan built directly from the checkpoint in that mode, and over the 21 int8 layers of the network it stays
    closer to the float result than the power-of-two plan (relative RMS, the reference's own error measure,
    test/common_utils.py:514-522 there)"""
    note("jit lowering, fractional scales")
    layers = nets.NETS["resnet18"]()
    x = torch.rand(2, 3, 64, 64, generator=torch.Generator().manual_seed(3))
    net, qnet = dropin_model(layers, x, 9, 0.05)
    fused, _ = jit.lower(qnet, x.cuda(), fractional_scale=True)
    pow2, _ = jit.lower(qnet, x.cuda())
    direct = pipeline.FusedNet(layers, pipeline.calibrate(net, x, "int8", True), fractional_scale=True)
    got = fused.forward(x.cuda())
    assert torch.equal(got, direct.forward(x.cuda()))
    from oracle import netref
    sd = pipeline.calibrate(net, x, "int8", True)
    t, _ = netref.run(layers, {k: v.detach().cpu().numpy() for k, v in sd.items()}, x.numpy(), record=False,
                      fractional_scale=True)
    assert np.array_equal(t[direct.outputs[0]].reshape(got.shape), got.cpu().numpy())
    ref = net(x).cuda()

    def rel_rms(a, b):
        return ((a - b).pow(2).sum().sqrt() / b.pow(2).sum().sqrt()).item()
    e_frac, e_pow2 = rel_rms(got, ref), rel_rms(pow2.forward(x.cuda()), ref)
    note("relative RMS vs float: fractional %.4f, power of two %.4f" % (e_frac, e_pow2))
    assert e_frac < e_pow2 <= 0.05


@pytest.mark.parametrize("arch,size,std", [("resnet18", 64, 0.05), ("mobilenet_v2", 64, 0.2),
                                           ("darknet53_yolov3", 64, "he")])
def test_lowered_trace_equals_direct_plan(arch, size, std):
    note("jit lowering", arch)
    layers = nets.NETS[arch]()
    x = torch.rand(2, 3, size, size, generator=torch.Generator().manual_seed(3))
    net, qnet = dropin_model(layers, x, 9, std)
    fused, lowered_layers = jit.lower(qnet, x.cuda())
    assert [l.kind for l in lowered_layers] == [l.kind for l in layers]
    for a, b in zip(lowered_layers, layers):
        assert (a.act, bool(a.add), bool(a.add and a.add_after), a.k, a.stride, a.pad, a.groups) == \
               (b.act, bool(b.add), bool(b.add and b.add_after), b.k, b.stride, b.pad, b.groups), (a, b)
    direct = pipeline.FusedNet(layers, pipeline.calibrate(net, x, "int8", True))
    got, want = fused.forward(x.cuda()), direct.forward(x.cuda())
    got = got if isinstance(got, tuple) else (got,)
    want = want if isinstance(want, tuple) else (want,)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert torch.equal(g, w)
    # against the oracle: the unfused network of the same checkpoint, run layer by layer on the CPU -- the lowered
    # plan's outputs are the oracle's bit for bit (fractional mode: test_lowering_with_fractional_scales)
    from oracle import netref
    sd = pipeline.calibrate(net, x, "int8", True)
    t, rec = netref.run(layers, {k: v.detach().cpu().numpy() for k, v in sd.items()}, x.numpy())
    assert all(r["overflow"] == 0 for r in rec.values())
    for name, g in zip(direct.outputs, got):  # the lowered plan names its tensors after the graph's nodes
        o = t[name]
        gn = g.cpu().numpy()
        gn = np.transpose(gn, (0, 2, 3, 1)) if gn.ndim == 4 else gn.reshape(o.shape)
        assert np.array_equal(o.reshape(gn.shape), gn), name
    # and the traced module itself (float tensors between the ops) agrees within the stated tolerance
    ref = qnet(x.cuda())
    ref = ref if isinstance(ref, tuple) else (ref,)
    for g, r in zip(got, ref):
        span = (r.max() - r.min()).item()
        assert (g - r).abs().max().item() <= 1e-3 * span + 1e-6


def test_lowering_rejects_unknown_nodes():
    note("jit lowering rejects")

    class Odd(torch.nn.Module):
        def __init__(self, inner):
            super().__init__()
            self.inner = inner

        def forward(self, x):
            return torch.sigmoid(self.inner(x))

    layers = nets.resnet(18)
    x = torch.rand(1, 3, 64, 64, generator=torch.Generator().manual_seed(4))
    _, qnet = dropin_model(layers, x, 2, 0.05)
    with pytest.raises(jit.LoweringError):
        jit.lower(Odd(qnet), x.cuda())

"""The entry point that allocates nothing (catchq_quantize_param_noalloc) against the entry point it is a
variant of (catchq_quantize_param), through the C ABI: bit-identical outputs on two calls in a row, the
second on a smaller input, so that whatever the first call left in the fixed scratch memory would show."""
import ctypes
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    import cabi


def _outputs(device):
    return (torch.full((1,), -1.0, dtype=torch.float32, device=device),
            torch.full((1,), -99, dtype=torch.int32, device=device),
            torch.full((1,), -1.0, dtype=torch.float32, device=device),
            torch.full((1,), -1.0, dtype=torch.float32, device=device))


def _noalloc(x, bw, mode=2):
    absmax, pos, scale, off = _outputs(x.device)
    cabi.check(cabi.lib().catchq_quantize_param_noalloc(cabi.ptr(x), cabi.dt(x), x.numel(), bw, mode, cabi.ptr(absmax),
                                                        cabi.ptr(pos), cabi.ptr(scale), cabi.ptr(off), cabi.stream()))
    return absmax, pos, scale, off


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_noalloc_equals_workspace_variant_on_two_calls_in_a_row(dtype):
    g = torch.Generator().manual_seed(11)
    # the first input fills all 4096 partial slots with large values; the second is small in size and in
    # magnitude, so a stale slot read by mistake would win the maximum
    big = (torch.randn(4096 * 4096 + 13, generator=g) * 50).to(dtype).cuda()
    small = (torch.randn(1000, generator=g) * 0.01).to(dtype).cuda()
    for bw in (8, 16):
        for x in (big, small):
            print("quantize_param_noalloc", dtype, bw, x.numel(), flush=True)
            sys.stdout.flush()
            got = _noalloc(x, bw)
            want = cabi.quantize_param(x, bw)
            for a, b in zip(got, want):
                assert torch.equal(a, b), (bw, x.numel(), a.item(), b.item())
            assert got[0].item() == x.float().abs().max().item()
    # modes that do not ask for scale / offset leave those outputs alone, like the variant with a workspace
    absmax, pos, scale, off = _noalloc(small, 8, mode=0)
    assert scale.item() == -1.0 and off.item() == -1.0 and pos.item() == cabi.quantize_param(small, 8)[1].item()


def test_noalloc_rejects_sizes_beyond_its_maximum_and_bad_arguments():
    x = torch.zeros(16, device="cuda")
    absmax, pos, scale, off = _outputs(x.device)
    lib = cabi.lib()
    too_many = (1 << 40) + 1
    st = lib.catchq_quantize_param_noalloc(cabi.ptr(x), 0, too_many, 8, 2, cabi.ptr(absmax), cabi.ptr(pos), cabi.ptr(scale),
                                           cabi.ptr(off), cabi.stream())
    assert st == 7 and b"scratch" in lib.catchq_status_string(st)
    assert lib.catchq_quantize_param_noalloc(cabi.ptr(x), 0, 16, 12, 2, cabi.ptr(absmax), cabi.ptr(pos), cabi.ptr(scale),
                                             cabi.ptr(off), cabi.stream()) == 3
    assert lib.catchq_quantize_param_noalloc(None, 0, 16, 8, 2, cabi.ptr(absmax), cabi.ptr(pos), cabi.ptr(scale),
                                             cabi.ptr(off), cabi.stream()) == 1
    torch.cuda.synchronize()
    assert pos.item() == -99   # nothing ran

"""The forward convolution + requantisation entry point that keeps its scratch memory inside the library
(niti_conv2d_i8_fprop_requant_static) against niti_conv2d_i8_fprop_requant, bit for bit, on calls in a row that share
the library's array - the second with a smaller input, so stale slots of the first would show."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ri8(g, *shape):
    return torch.randint(-127, 128, shape, generator=g, dtype=torch.int8)


def test_static_scratch_entry_matches_the_caller_scratch_entry():
    from niti_amd import _lib as L
    from niti_amd import ops
    from oracle import niti_oracle as po
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(707)
    assert L.lib().niti_static_scratch_bytes() <= 5 << 20
    # large first (512 workgroups, a 144 KB filter copy), then smaller ones, then the first again
    shapes = [(64, 32, 32, 64, 128), (4, 16, 16, 32, 48), (16, 4, 4, 16, 16), (4, 8, 8, 16, 32), (64, 32, 32, 64, 128)]
    for i, (N, H, W, C, K) in enumerate(shapes):
        print("static", i, (N, H, W, C, K), flush=True)
        x, w = _ri8(g, N, H, W, C), _ri8(g, K, 3, 3, C)
        if i == 2:
            x = torch.randint(-3, 4, x.shape, generator=g, dtype=torch.int8)   # small sums: another shift than the call before
        xd, wd = x.to(dev), w.to(dev)
        for relu, method, dm in ((False, "round", "floor"), (True, "psto", "trunc")):
            ref, ref_shift, ref_sync = ops.conv2d_fprop_requant(xd, wd, method=method, div_mode=dm, relu=relu, f32_epilogue=True)
            e_a = torch.tensor([-3], dtype=torch.int32, device=dev)
            e_out = torch.zeros(1, dtype=torch.int32, device=dev)
            rng = torch.full((2,), -1, dtype=torch.int32, device=dev)
            y, shift = ops.conv2d_fprop_requant_static(xd, wd, method=method, div_mode=dm, relu=relu, f32_epilogue=True, exp_a=e_a,
                                                       exp_out=e_out, range_out=rng)
            torch.cuda.synchronize()
            assert torch.equal(y, ref), (i, relu, method)
            assert int(shift) == int(ref_shift) and int(e_out) == int(ref_shift) - 3
            assert int(rng[0]) == int(ref_sync[0]) and int(rng[1]) == 0
        # and against the CPU oracle
        acc = po.conv2d_int8(x, w, 1, 1, True)
        want, _ = po.act_calc(acc, 0, "round", "floor")
        y, _ = ops.conv2d_fprop_requant_static(xd, wd, f32_epilogue=True)
        assert torch.equal(y.cpu(), want), i
    # a prepared filter needs no room in the library's array
    N, H, W, C, K = 4, 8, 8, 16, 32
    x, w = _ri8(g, N, H, W, C), _ri8(g, K, 3, 3, C)
    wp = ops.conv_filter_prepare(w.to(dev), N, H, W)
    ref, _, _ = ops.conv2d_fprop_requant(x.to(dev), w.to(dev))
    y, _ = ops.conv2d_fprop_requant_static(x.to(dev), w.to(dev), prepared_filter=wp)
    assert torch.equal(y, ref)


def test_static_scratch_entry_refuses_what_does_not_fit():
    from niti_amd import _lib as L
    from niti_amd import ops
    dev = torch.device("cuda:0")
    # filter copy of 1024 x 9 x 1024 bytes: beyond the 4 MiB the library holds
    x = torch.zeros((16, 4, 4, 1024), dtype=torch.int8, device=dev)
    w = torch.zeros((1024, 3, 3, 1024), dtype=torch.int8, device=dev)
    with pytest.raises(L.NitiError, match="static scratch holds"):
        ops.conv2d_fprop_requant_static(x, w)
    # a shape outside the single-launch path
    x = torch.zeros((2, 9, 9, 16), dtype=torch.int8, device=dev)
    w = torch.zeros((16, 3, 3, 16), dtype=torch.int8, device=dev)
    with pytest.raises(L.NitiError, match="not covered"):
        ops.conv2d_fprop_requant_static(x, w)

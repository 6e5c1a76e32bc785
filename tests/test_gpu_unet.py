"""The gated-convolution U-Net forward on the matrix cores against a plain-torch fp32 restatement.

Tolerance: operands are fp16 (weights, block inputs, activations between blocks), accumulation fp32. The torch
restatement rounds at the same places, so what remains is summation order inside a 9 x Cin dot product and the fast
exp of the device epilogue: 2e-3 of the largest output magnitude. Against the unrounded fp32 network the bar is the
fp16 one, 2e-2."""
import numpy as np
import pytest
import torch

from trips_amd import abi

pytestmark = pytest.mark.gpu


def _pyramid(w, h, levels, channels, batch, seed):
    g = torch.Generator().manual_seed(seed)
    sizes = abi.layer_sizes(w, h, levels)
    return [torch.rand((batch, channels, hh, ww), generator=g) for (ww, hh) in sizes]


def _net(filters, levels, seed, cin=4):
    from trips_amd.unet import MultiScaleUnet2dDecOnlySmallFixed, MultiScaleUnet2dParams
    p = MultiScaleUnet2dParams(num_input_layers=levels, num_layers=levels, num_input_channels=cin,
                               filters_network=list(filters))
    net = MultiScaleUnet2dDecOnlySmallFixed(p)
    g = torch.Generator().manual_seed(seed)
    net.he_normal_(g)
    with torch.no_grad():
        for m in net.modules():
            if isinstance(m, torch.nn.Conv2d):
                m.bias.normal_(0.0, 0.1, generator=g)
    return net


def _compare(net, inputs, tol_rounded=2e-3, tol_fp32=2e-2):
    from tests.ref_unet import unet_forward
    with torch.no_grad():
        want = unet_forward(net, inputs, half_rounding=True).numpy()
        want32 = unet_forward(net, inputs, half_rounding=False).numpy()
        got = net.forward([t.cuda() for t in inputs]).cpu().numpy()
    assert got.shape == want.shape
    scale = np.abs(want).max()
    assert np.abs(got - want).max() < tol_rounded * scale, np.abs(got - want).max() / scale
    assert np.abs(got - want32).max() < tol_fp32 * scale


@pytest.mark.parametrize("filters,levels,w,h", [
    ([16, 32, 64, 64], 4, 96, 72),      # the benchmark's channel plan; sizes halve exactly
    ([32, 32, 32, 32, 32], 5, 100, 60),  # the shipped configuration's filters; odd sizes -> centre crop
    ([16, 24], 2, 37, 29),               # partial tiles everywhere
    ([20], 1, 40, 24),                   # start block only
    ([32, 64, 64], 3, 70, 50),           # 64 input channels at the finest level, whose kernel also holds the 1x1
    ([16, 48, 32], 3, 70, 50),           # 40 outputs on 32 inputs: the one shape whose weight gradient runs four wavefronts
])
def test_unet_forward_matches_torch(filters, levels, w, h):
    net = _net(filters, levels, seed=levels)
    inputs = _pyramid(w, h, levels, 4, batch=2, seed=10 + levels)
    if levels == 1:
        # a one-level net feeds the final 1x1 with F[0] - C channels; the reference's final expects F[0]
        net.final = torch.nn.Sequential(torch.nn.Conv2d(filters[0] - 4, 3, 1), torch.nn.Identity())
    _compare(net, inputs)


def test_unet_forward_three_input_channels():
    net = _net([16, 32, 32], 3, seed=5, cin=3)
    inputs = _pyramid(64, 48, 3, 3, batch=1, seed=6)
    _compare(net, inputs)


@pytest.mark.parametrize("cin,filters,levels,w,h", [
    (6, [24, 32, 64], 3, 70, 50),        # the coarser level's outputs start at position 12 of the finer block's input
    (8, [32, 48, 64, 64], 4, 96, 72),    # ... at 16
    (16, [48, 64, 64], 3, 70, 50),       # ... at 32: the image fills the first two groups of eight
    (16, [40], 1, 40, 24),               # start block only
])
def test_unet_forward_more_input_channels(cin, filters, levels, w, h):
    """The descriptor widths of the splat beyond four (6, 8, 16 channels per image)."""
    net = _net(filters, levels, seed=40 + cin, cin=cin)
    inputs = _pyramid(w, h, levels, cin, batch=2, seed=50 + cin)
    if levels == 1:
        net.final = torch.nn.Sequential(torch.nn.Conv2d(filters[0] - cin, 3, 1), torch.nn.Identity())
    _compare(net, inputs)


def test_unet_packed_weights_are_reused_on_request():
    """A viewer's frames: with reuse_packed_weights the fp16 weights are packed by the first no-grad forward only
    (TripsUnetDesc.weights_packed); the later frames give the same bits, and a changed weight takes effect after
    invalidate_packed_weights()."""
    from trips_amd.renderer import get_context
    net = _net([16, 32, 64, 64], 4, seed=3).cuda()
    inputs = [t.cuda() for t in _pyramid(96, 72, 4, 4, batch=1, seed=4)]
    ctx = get_context(0)
    with torch.no_grad():
        ctx.profile_enable(True)
        ctx.profile_read()
        first = net.forward(inputs).clone()  # packs
        names_first = set(ctx.profile_read())
        net.reuse_packed_weights = True
        a = net.forward(inputs).clone()      # reuses what the call before left in the workspace
        names_a = set(ctx.profile_read())
        b = net.forward(inputs).clone()
        names_b = set(ctx.profile_read())
        assert "unet_pack_weights" in names_first and "unet_conv_l0" in names_b
        assert "unet_pack_weights" not in names_a and "unet_pack_weights" not in names_b
        assert torch.equal(first, a) and torch.equal(a, b)
        other = [t * 0.5 for t in inputs]
        assert torch.equal(net.forward(other), _fresh_forward(net, other))  # other inputs, same weights: still reused
        net.final_conv.bias.add_(1.0)
        net.block(1).feature_conv.weight.mul_(2.0)
        net.invalidate_packed_weights()
        c = net.forward(inputs).clone()
        names_c = set(ctx.profile_read())
        ctx.profile_enable(False)
        assert "unet_pack_weights" in names_c
        assert not torch.equal(c, a) and torch.equal(c, _fresh_forward(net, inputs))


def _fresh_forward(net, inputs):
    """The same forward with the packing done by the call itself."""
    keep, net.reuse_packed_weights = net.reuse_packed_weights, False
    try:
        return net.forward(inputs).clone()
    finally:
        net.reuse_packed_weights = keep
        net.invalidate_packed_weights()


def test_unet_extra_input_layers_are_ignored():
    # the splat renders 8 layers, the net may consume fewer (num_input_layers > num_layers)
    from trips_amd.unet import MultiScaleUnet2dDecOnlySmallFixed, MultiScaleUnet2dParams
    p = MultiScaleUnet2dParams(num_input_layers=4, num_layers=2, filters_network=[16, 32])
    net = MultiScaleUnet2dDecOnlySmallFixed(p).he_normal_(torch.Generator().manual_seed(1))
    inputs = _pyramid(64, 32, 4, 4, batch=1, seed=2)
    from tests.ref_unet import unet_forward
    with torch.no_grad():
        want = unet_forward(net, inputs).numpy()
        got = net.forward([t.cuda() for t in inputs]).cpu().numpy()
    assert np.abs(got - want).max() < 2e-3 * np.abs(want).max()


def test_unet_refuses_cpu_tensors():
    net = _net([16, 32], 2, seed=1)
    inputs = _pyramid(32, 32, 2, 4, batch=1, seed=2)
    with torch.no_grad(), pytest.raises(RuntimeError):
        net.forward(inputs)


# Gradients: fp16 operands in every GEMM of the backward as well (pre-activation gradients, block-input gradients),
# fp32 accumulation; compared with torch autograd through the restatement that rounds where the forward rounds.
# Bar: 2e-2 of the largest magnitude of each gradient tensor.
GRAD_TOL = 2e-2


@pytest.mark.parametrize("filters,levels,w,h,batch,cin", [
    ([16, 32, 64, 64], 4, 96, 72, 1, 4),      # the benchmark's channel plan
    ([32, 32, 32, 32, 32], 5, 100, 60, 2, 4),  # shipped filters, odd sizes, two images
    ([16, 24], 2, 37, 29, 1, 4),               # partial tiles
    ([32, 64, 64], 3, 70, 50, 1, 4),           # 64 input channels at the finest level
    ([16, 48, 32], 3, 70, 50, 2, 4),           # 40 outputs on 32 inputs (the weight gradient's four-wavefront shape)
    # fewer than four image channels: the coarser level's outputs then start at a position of the finer block's input
    # that is not a multiple of eight
    ([16, 32, 64, 64], 4, 96, 72, 1, 3),       # 58 outputs below 64 inputs: no spare position
    ([16, 24, 32], 3, 37, 29, 2, 2),
    ([12, 20], 2, 40, 24, 1, 1),
    # the splat's other descriptor widths: the image then spans up to two groups of eight positions
    ([24, 32, 64], 3, 70, 50, 1, 6),
    ([32, 48, 64, 64], 4, 96, 72, 2, 8),
    ([48, 64, 64], 3, 70, 50, 1, 16),
    ([40, 56], 2, 37, 29, 1, 12),               # (a width the splat does not have: 24 positions of image)
])
def test_unet_backward_matches_torch_autograd(filters, levels, w, h, batch, cin):
    import copy
    from tests.ref_unet import unet_forward
    net = _net(filters, levels, seed=20 + levels, cin=cin)
    ref = copy.deepcopy(net)
    inputs = _pyramid(w, h, levels, cin, batch=batch, seed=30 + levels)
    g = torch.Generator().manual_seed(7)
    upstream = torch.randn((batch, 3, h, w), generator=g) * 1e-3

    ins_ref = [t.clone().requires_grad_(True) for t in inputs]
    (unet_forward(ref, ins_ref, half_rounding=True) * upstream).sum().backward()

    net = net.cuda()
    ins = [t.cuda().requires_grad_(True) for t in inputs]
    out = net.forward(ins)
    (out * upstream.cuda()).sum().backward()

    def check(name, got, want):
        got, want = got.detach().cpu().numpy(), want.detach().numpy()
        scale = np.abs(want).max()
        err = np.abs(got - want).max()
        assert err < GRAD_TOL * scale, f"{name}: {err / scale:.3e}"

    for i in range(levels):
        check(f"d inputs[{i}]", ins[i].grad, ins_ref[i].grad)
    for (n1, p1), (n2, p2) in zip(net.named_parameters(), ref.named_parameters()):
        assert n1 == n2
        check(n1, p1.grad, p2.grad)


def test_unet_backward_small_gradients_survive_fp16():
    """dL/doutput of a mean loss over a full-HD image is ~1e-7, below fp16's smallest normal number: the scale the
    gradients are carried with must keep them."""
    import copy
    from tests.ref_unet import unet_forward
    net = _net([16, 32], 2, seed=3)
    ref = copy.deepcopy(net)
    inputs = _pyramid(64, 48, 2, 4, batch=1, seed=4)
    upstream = torch.full((1, 3, 48, 64), 1.0 / 6_220_800)
    ins_ref = [t.clone().requires_grad_(True) for t in inputs]
    # the unrounded fp32 network: torch's own fp16 casts would flush these gradients in the restatement itself
    (unet_forward(ref, ins_ref, half_rounding=False) * upstream).sum().backward()
    net = net.cuda()
    ins = [t.cuda().requires_grad_(True) for t in inputs]
    (net.forward(ins) * upstream.cuda()).sum().backward()
    for a, b in zip(ins, ins_ref):
        want = b.grad.numpy()
        assert np.abs(want).max() < 1e-6
        assert np.abs(a.grad.cpu().numpy() - want).max() < 3e-2 * np.abs(want).max()
    want = ref.up1.convolution.feature_conv.weight.grad.numpy()
    assert np.abs(net.up1.convolution.feature_conv.weight.grad.cpu().numpy() - want).max() < 3e-2 * np.abs(want).max()

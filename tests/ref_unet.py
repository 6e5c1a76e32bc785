"""Plain-torch restatement of the reference's decoder-only U-Net forward (src/lib/models/Networks.h:751-787,
999-1208 of the reference: SmallDecStartBlock, UpsampleDecOnlySmallBlockFixed, MultiScaleUnet2dDecOnlySmallFixed)
for bilinear upsampling, gated blocks, elu, no norm, identity last activation. Test infrastructure: the checker
for the HIP net, never the product.

`half_rounding=True` rounds to fp16 wherever the device path stores or feeds fp16 (weights, convolution inputs,
activations between blocks), so that what is left between the two is accumulation order and exp() accuracy.
"""
import torch
import torch.nn.functional as F


def _r(t, on):
    return t.half().float() if on else t


def _center_crop(t, h, w):
    dh, dw = t.shape[2] - h, t.shape[3] - w
    return t[:, :, dh // 2:dh // 2 + h, dw // 2:dw // 2 + w]


def gated(x, blk, half_rounding):
    wf, bf = _r(blk.feature_conv.weight, half_rounding), blk.feature_conv.bias
    wm, bm = _r(blk.mask_conv.weight, half_rounding), blk.mask_conv.bias
    x = _r(x, half_rounding)
    f = F.elu(F.conv2d(x, wf, bf, padding=1))
    m = torch.sigmoid(F.conv2d(x, wm, bm, padding=1))
    return _r(f * m, half_rounding)


def unet_forward(net, inputs, half_rounding=True):
    """net: trips_amd.unet.MultiScaleUnet2dDecOnlySmallFixed (parameters only are used); inputs: CPU fp32 list."""
    p = net.params
    L = p.num_layers
    net = net.float()
    x = inputs[L - 1]
    cur = torch.cat([_r(x, half_rounding), gated(x, net.block(L - 1), half_rounding)], 1)
    for i in range(L - 2, -1, -1):
        up = F.interpolate(cur, scale_factor=2.0, mode="bilinear", align_corners=False)
        feats = inputs[i]
        up = _center_crop(up, feats.shape[2], feats.shape[3])
        comb = torch.cat([feats, up], 1)
        cur = torch.cat([_r(feats, half_rounding), gated(comb, net.block(i), half_rounding)], 1)
    return F.conv2d(cur, _r(net.final_conv.weight, half_rounding), net.final_conv.bias)

"""Host-side mirror of the reference's reconstruction net over the C ABI of include/trips_unet.h.

Names follow src/lib/models/Networks.h of the reference: MultiScaleUnet2dParams (:Pipeline ini section
[MultiScaleUnet2dParams], configs/train_normalnet.ini:200-219) and MultiScaleUnet2dDecOnlySmallFixed
(Networks.h:1080-1208) with the registered module names `start`, `up1` .. `up<L-1>`, `final`. The gated block's
own parameter names come from an un-vendored dependency; `feature_transform` / `mask_transform` are used here.

Inference only: forward() runs the HIP kernels (fp16 operands on the matrix cores); there is no CPU path and no
backward yet (forward() refuses inputs or weights that require grad inside an autograd-enabled region).
"""
import ctypes as C
import math
from dataclasses import dataclass, field
from typing import List

import torch

from . import _lib, abi
from .renderer import _ptr, _stream_ptr, get_context


@dataclass
class MultiScaleUnet2dParams:
    num_input_layers: int = 5
    num_input_channels: int = 4
    num_output_channels: int = 3
    num_layers: int = 5
    half_float: bool = False  # the device path always runs fp16 operands with fp32 accumulation
    upsample_mode: str = "bilinear"
    norm_layer_up: str = "id"
    last_act: str = "id"
    conv_block_up: str = "gated"
    activation: str = "elu"
    network_version: str = "MultiScaleUnet2dDecOnlySmallFixed"
    filters_network: List[int] = field(default_factory=lambda: [32] * 8)


class GatedBlock(torch.nn.Module):
    """elu(conv_f(x)) * sigmoid(conv_m(x)), 3x3, stride 1, zero padding 1; holds the parameters only."""

    def __init__(self, in_channels, out_channels):
        super().__init__()
        self.feature_transform = torch.nn.Conv2d(in_channels, out_channels, 3, padding=1)
        self.mask_transform = torch.nn.Conv2d(in_channels, out_channels, 3, padding=1)


class MultiScaleUnet2dDecOnlySmallFixed(torch.nn.Module):
    def __init__(self, params: MultiScaleUnet2dParams):
        super().__init__()
        p = params
        for name, want in (("upsample_mode", "bilinear"), ("norm_layer_up", "id"), ("last_act", "id"),
                           ("conv_block_up", "gated"), ("activation", "elu")):
            if getattr(p, name) != want:
                raise NotImplementedError(f"MultiScaleUnet2dParams.{name} = {getattr(p, name)!r}: only {want!r} is built")
        if p.num_input_layers < p.num_layers:
            raise ValueError("num_input_layers < num_layers")
        self.params = p
        L, Cin, F = p.num_layers, p.num_input_channels, list(p.filters_network)
        # Networks.h:1104-1118: start block outputs F[L-1] - 2C, block i outputs F[i] - 2C (F[0] - C for the last)
        self.start = GatedBlock(Cin, F[L - 1] - 2 * Cin)
        for i in range(L - 2, -1, -1):
            out = F[i] - (Cin if i == 0 else 2 * Cin)
            self.add_module(f"up{i + 1}", GatedBlock(F[i + 1], out))
        self.final = torch.nn.Conv2d(F[0], p.num_output_channels, 1)
        self._workspace = None

    def block(self, i):
        """Gated block of pyramid level i (the start block for the coarsest level)."""
        L = self.params.num_layers
        return self.start if i == L - 1 else getattr(self, f"up{i + 1}")

    def he_normal_(self, generator=None):
        """He-normal weights, zero biases (the initialisation the benchmark configuration names)."""
        for m in self.modules():
            if isinstance(m, torch.nn.Conv2d):
                fan_in = m.in_channels * m.kernel_size[0] * m.kernel_size[1]
                with torch.no_grad():
                    m.weight.normal_(0.0, math.sqrt(2.0 / fan_in), generator=generator)
                    m.bias.zero_()
        return self

    def desc(self, inputs):
        p = self.params
        sizes = [(int(t.shape[3]), int(t.shape[2])) for t in inputs[:p.num_layers]]
        return abi.make_unet_desc(p.filters_network, sizes, p.num_input_channels, p.num_output_channels,
                                  batch=int(inputs[0].shape[0]))

    def forward(self, inputs, masks=None):
        """inputs: the splat's image pyramid, [B, C, H_l, W_l] fp32 per level, finest first. Returns [B, 3, H, W]."""
        p = self.params
        if len(inputs) != p.num_input_layers:
            raise ValueError(f"{len(inputs)} input layers, params.num_input_layers = {p.num_input_layers}")
        if torch.is_grad_enabled() and (any(t.requires_grad for t in inputs) or
                                        any(q.requires_grad for q in self.parameters())):
            raise NotImplementedError("the device net is inference only: call it under torch.no_grad()")
        dev = inputs[0].device
        if dev.type != "cuda":
            raise RuntimeError("MultiScaleUnet2dDecOnlySmallFixed needs GPU tensors: there is no CPU implementation")
        ctx = get_context(dev.index or 0)
        L = p.num_layers
        ins = []
        for i in range(L):
            t = inputs[i]
            if t.dtype != torch.float32 or t.shape[1] != p.num_input_channels:
                raise ValueError(f"inputs[{i}]: expected float32 [B, {p.num_input_channels}, H, W]")
            ins.append(t.contiguous())
        d = self.desc(ins)
        w = abi.TripsUnetWeights()
        keep = []
        for i in range(L):
            blk = self.block(i)
            for name, conv_attr, field_ in (("feature_weight", "feature_transform", "weight"),
                                            ("feature_bias", "feature_transform", "bias"),
                                            ("mask_weight", "mask_transform", "weight"),
                                            ("mask_bias", "mask_transform", "bias")):
                t = getattr(getattr(blk, conv_attr), field_).detach().to(dev, torch.float32).contiguous()
                keep.append(t)
                getattr(w, name)[i] = t.data_ptr()
        fw = self.final.weight.detach().to(dev, torch.float32).contiguous()
        fb = self.final.bias.detach().to(dev, torch.float32).contiguous()
        w.final_weight, w.final_bias = fw.data_ptr(), fb.data_ptr()
        nbytes = C.c_size_t(0)
        _lib.check(ctx.lib.trips_unet_workspace_size(C.byref(d), C.byref(nbytes)))
        if self._workspace is None or self._workspace.numel() < nbytes.value or self._workspace.device != dev:
            self._workspace = ctx.alloc_bytes(nbytes.value)
        out = torch.empty((d.batch, p.num_output_channels, d.level_h[0], d.level_w[0]), dtype=torch.float32, device=dev)
        ptrs = (C.c_void_p * abi.TRIPS_UNET_MAX_LEVELS)()
        for i in range(L):
            ptrs[i] = ins[i].data_ptr()
        _lib.check(ctx.lib.trips_unet_forward(ctx.ctx, C.byref(d), C.byref(w), ptrs, _ptr(out), _ptr(self._workspace),
                                              nbytes.value, _stream_ptr(dev)))
        return out

    def flops(self, inputs):
        d = self.desc(inputs)
        f = C.c_double(0)
        _lib.check(_lib.load().trips_unet_flops(C.byref(d), C.byref(f)))
        return float(f.value)

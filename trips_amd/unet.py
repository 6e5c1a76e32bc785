"""Host-side mirror of the reference's reconstruction net over the C ABI of include/trips_unet.h.

Names follow src/lib/models/Networks.h of the reference: MultiScaleUnet2dParams (ini section
[MultiScaleUnet2dParams], configs/train_normalnet.ini:200-219) and MultiScaleUnet2dDecOnlySmallFixed
(Networks.h:1080-1208) with the registered module names `start.conv`, `up<i>.up`, `up<i>.convolution`, `final`.
The gated block's own parameter names come from an un-vendored dependency; Sequentials `feature_transform` /
`mask_transform` (convolution at index 0) are used here.

forward() runs the HIP kernels (fp16 operands on the matrix cores, fp32 accumulation); with autograd enabled it
records one graph node whose backward is the device backward. There is no CPU path.
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
    """elu(conv_f(x)) * sigmoid(conv_m(x)), 3x3, stride 1, zero padding 1; holds the parameters only.
    The two branches are Sequentials (convolution, activation), so a parameter is `feature_transform.0.weight`."""

    def __init__(self, in_channels, out_channels):
        super().__init__()
        self.feature_transform = torch.nn.Sequential(torch.nn.Conv2d(in_channels, out_channels, 3, padding=1), torch.nn.ELU())
        self.mask_transform = torch.nn.Sequential(torch.nn.Conv2d(in_channels, out_channels, 3, padding=1), torch.nn.Sigmoid())

    @property
    def feature_conv(self):
        return self.feature_transform[0]

    @property
    def mask_conv(self):
        return self.mask_transform[0]


class SmallDecStartBlock(torch.nn.Module):
    """Networks.h:751-787: registers its gated block as `conv`."""

    def __init__(self, in_channels, out_channels):
        super().__init__()
        self.conv = GatedBlock(in_channels, out_channels)


class UpsampleDecOnlySmallBlockFixed(torch.nn.Module):
    """Networks.h:999-1098: registers `up` (the bilinear upsampling) and `convolution` (the gated block)."""

    def __init__(self, in_channels, conv_out_channels):
        super().__init__()
        self.up = torch.nn.Sequential(torch.nn.Upsample(scale_factor=2.0, mode="bilinear", align_corners=False))
        self.convolution = GatedBlock(in_channels, conv_out_channels)


class _UnetFunction(torch.autograd.Function):
    """One graph node for the whole net: inputs (pyramid levels) and parameters in, image out."""

    @staticmethod
    def forward(ctx_, net, n_levels, *tensors):
        ins = [t.detach() for t in tensors[:n_levels]]
        params = [t.detach() for t in tensors[n_levels:]]
        saved = net._alloc("saved", net._size("trips_unet_saved_size", ins), ins[0].device)
        out = net._run_forward(ins, params, saved)
        ctx_.net, ctx_.ins, ctx_.params, ctx_.saved = net, ins, params, saved
        return out

    @staticmethod
    def backward(ctx_, d_out):
        net = ctx_.net
        d_ins, d_params = net._run_backward(ctx_.ins, ctx_.params, ctx_.saved, d_out.contiguous().float())
        return (None, None, *d_ins, *d_params)


class MultiScaleUnet2dDecOnlySmallFixed(torch.nn.Module):
    def __init__(self, params: MultiScaleUnet2dParams, grad_scale: float = 65536.0):
        super().__init__()
        p = params
        for name, want in (("upsample_mode", "bilinear"), ("norm_layer_up", "id"), ("last_act", "id"),
                           ("conv_block_up", "gated"), ("activation", "elu")):
            if getattr(p, name) != want:
                raise NotImplementedError(f"MultiScaleUnet2dParams.{name} = {getattr(p, name)!r}: only {want!r} is built")
        if p.num_input_layers < p.num_layers:
            raise ValueError("num_input_layers < num_layers")
        self.params = p
        self.grad_scale = float(grad_scale)  # factor the fp16 gradients inside the backward are carried with
        L, Cin, F = p.num_layers, p.num_input_channels, list(p.filters_network)
        # Networks.h:1104-1118: start block outputs F[L-1] - 2C, block i outputs F[i] - 2C (F[0] - C for the last)
        self.start = SmallDecStartBlock(Cin, F[L - 1] - 2 * Cin)
        for i in range(L - 2, -1, -1):
            out = F[i] - (Cin if i == 0 else 2 * Cin)
            self.add_module(f"up{i + 1}", UpsampleDecOnlySmallBlockFixed(F[i + 1], out))
        self.final = torch.nn.Sequential(torch.nn.Conv2d(F[0], p.num_output_channels, 1), torch.nn.Identity())
        self._buffers_dev = {}
        # A viewer sets this: the weights then count as unchanged from one no-grad forward to the next (they are packed
        # to fp16 once, not per frame). Whoever changes them in place afterwards (load_state_dict, an optimiser step)
        # calls invalidate_packed_weights().
        self.reuse_packed_weights = False
        self._packed_key = None

    def invalidate_packed_weights(self):
        self._packed_key = None

    def block(self, i):
        """Gated block of pyramid level i (the start block's for the coarsest level)."""
        L = self.params.num_layers
        return self.start.conv if i == L - 1 else getattr(self, f"up{i + 1}").convolution

    @property
    def final_conv(self):
        return self.final[0]

    def ordered_parameters(self):
        """Parameters in the order of the C structs: per level feature weight, bias, mask weight, bias; then final."""
        out = []
        for i in range(self.params.num_layers):
            b = self.block(i)
            out += [b.feature_conv.weight, b.feature_conv.bias, b.mask_conv.weight, b.mask_conv.bias]
        return out + [self.final_conv.weight, self.final_conv.bias]

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

    # ---- plumbing ----
    def _size(self, fn, inputs):
        d = self.desc(inputs)
        n = C.c_size_t(0)
        _lib.check(getattr(_lib.load(), fn)(C.byref(d), C.byref(n)))
        return int(n.value)

    def _alloc(self, key, nbytes, dev):
        if key == "saved":  # one per forward: a later forward must not overwrite what an earlier graph still needs
            return get_context(dev.index or 0).alloc_bytes(nbytes)
        buf = self._buffers_dev.get(key)
        if buf is None or buf.numel() < nbytes or buf.device != dev:
            buf = get_context(dev.index or 0).alloc_bytes(nbytes)
            self._buffers_dev[key] = buf
        return buf

    def _weights_struct(self, params):
        w = abi.TripsUnetWeights()
        L = self.params.num_layers
        for i in range(L):
            w.feature_weight[i], w.feature_bias[i] = params[4 * i].data_ptr(), params[4 * i + 1].data_ptr()
            w.mask_weight[i], w.mask_bias[i] = params[4 * i + 2].data_ptr(), params[4 * i + 3].data_ptr()
        w.final_weight, w.final_bias = params[4 * L].data_ptr(), params[4 * L + 1].data_ptr()
        return w

    @staticmethod
    def _input_ptrs(ins):
        ptrs = (C.c_void_p * abi.TRIPS_UNET_MAX_LEVELS)()
        for i, t in enumerate(ins):
            ptrs[i] = t.data_ptr()
        return ptrs

    def _run_forward(self, ins, params, saved):
        dev = ins[0].device
        ctx = get_context(dev.index or 0)
        d = self.desc(ins)
        w = self._weights_struct(params)
        nbytes = self._size("trips_unet_workspace_size", ins)
        ws = self._alloc("forward", nbytes, dev)
        # the packed weights in the workspace stay valid while the weights do (reuse_packed_weights), for the same
        # buffer and level sizes
        key = (ws.data_ptr(), bytes(d), tuple(q.data_ptr() for q in params))
        if self.reuse_packed_weights and saved is None and self._packed_key == key:
            d.weights_packed = 1
        self._packed_key = key if saved is None else None
        out = torch.empty((d.batch, d.num_output_channels, d.level_h[0], d.level_w[0]), dtype=torch.float32, device=dev)
        _lib.check(ctx.lib.trips_unet_forward(ctx.ctx, C.byref(d), C.byref(w), self._input_ptrs(ins), _ptr(out),
                                              _ptr(saved), _ptr(ws), nbytes, _stream_ptr(dev)))
        return out

    def _run_backward(self, ins, params, saved, d_out):
        dev = ins[0].device
        ctx = get_context(dev.index or 0)
        d = self.desc(ins)
        w = self._weights_struct(params)
        nbytes = self._size("trips_unet_backward_workspace_size", ins)
        ws = self._alloc("backward", nbytes, dev)
        L = self.params.num_layers
        g = abi.TripsUnetGrads()
        d_params = [torch.empty_like(t) for t in params]
        d_ins = [torch.empty_like(t) for t in ins]
        for i in range(L):
            g.feature_weight[i], g.feature_bias[i] = d_params[4 * i].data_ptr(), d_params[4 * i + 1].data_ptr()
            g.mask_weight[i], g.mask_bias[i] = d_params[4 * i + 2].data_ptr(), d_params[4 * i + 3].data_ptr()
            g.inputs[i] = d_ins[i].data_ptr()
        g.final_weight, g.final_bias = d_params[4 * L].data_ptr(), d_params[4 * L + 1].data_ptr()
        _lib.check(ctx.lib.trips_unet_backward(ctx.ctx, C.byref(d), C.byref(w), self._input_ptrs(ins), _ptr(saved),
                                               _ptr(d_out), C.c_float(self.grad_scale), C.byref(g), _ptr(ws), nbytes,
                                               _stream_ptr(dev)))
        return d_ins, d_params

    # ---- the reference's call ----
    def forward(self, inputs, masks=None):
        """inputs: the splat's image pyramid, [B, C, H_l, W_l] fp32 per level, finest first. Returns [B, 3, H, W]."""
        p = self.params
        if len(inputs) != p.num_input_layers:
            raise ValueError(f"{len(inputs)} input layers, params.num_input_layers = {p.num_input_layers}")
        dev = inputs[0].device
        if dev.type != "cuda":
            raise RuntimeError("MultiScaleUnet2dDecOnlySmallFixed needs GPU tensors: there is no CPU implementation")
        L = p.num_layers
        ins = []
        for i in range(L):
            t = inputs[i]
            if t.dtype != torch.float32 or t.shape[1] != p.num_input_channels:
                raise ValueError(f"inputs[{i}]: expected float32 [B, {p.num_input_channels}, H, W]")
            ins.append(t.contiguous())
        params = [q.to(dev, torch.float32).contiguous() for q in self.ordered_parameters()]
        needs_grad = torch.is_grad_enabled() and (any(t.requires_grad for t in ins) or any(q.requires_grad for q in params))
        if needs_grad:
            return _UnetFunction.apply(self, L, *ins, *params)
        return self._run_forward([t.detach() for t in ins], [q.detach() for q in params], None)

    def flops(self, inputs):
        d = self.desc(inputs)
        f = C.c_double(0)
        _lib.check(_lib.load().trips_unet_flops(C.byref(d), C.byref(f)))
        return float(f.value)

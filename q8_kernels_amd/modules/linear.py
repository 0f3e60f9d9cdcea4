"""Q8Linear / Q8LinearLora / FP8Linear modules (reference: q8_kernels/modules/linear.py:11-146).

State-dict layout is the reference's: `weight` (int8 or e4m3, [out, in], already rotated when
quantized with Hadamard), `scales` (fp32 [out], buffer) and `bias` (fp32 [out])."""
import torch
import torch.nn as nn

from .. import functional as Q8F


def _is_16bit(t) -> bool:
    return t.dtype in (torch.float16, torch.bfloat16)


class _QuantLinearBase(nn.Module):
    weight_dtype = torch.int8

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.empty(out_features, in_features, device=device, dtype=self.weight_dtype),
                                   requires_grad=False)
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features, device=device, dtype=torch.float), requires_grad=False)
        else:
            self.register_parameter("bias", None)
        self.register_buffer("scales", torch.empty(out_features, device=device, dtype=torch.float))

    def _bias(self):
        return None if self.bias is None else self.bias.data

    def _adopt(self, w_quant, w_scale, linear):
        self.weight.data = w_quant
        self.scales.data = w_scale
        if linear.bias is not None:
            self.bias.data = linear.bias.data.float()
        return self


class Q8Linear(_QuantLinearBase):
    """int8 weights; activations are FHT-rotated and int8-quantized per token inside forward."""
    weight_dtype = torch.int8

    def forward(self, x, x_scales=None, fuse_gelu=False, out_dtype=None, residual=None, gate=None):
        return Q8F.linear.q8_linear(x, self.weight.data, self._bias(), x_scales, self.scales, fuse_gelu, out_dtype,
                                    residual, gate)

    @classmethod
    def from_linear(cls, linear: nn.Linear, quant_with_hadamard=True):
        w = linear.weight.data
        assert w.is_cuda, "input linear layer must be in cuda device"
        assert w.dtype == torch.float8_e4m3fn or _is_16bit(w)
        layer = cls(linear.in_features, linear.out_features, linear.bias is not None, w.device)
        if quant_with_hadamard:
            w = Q8F.fast_hadamard.hadamard_transform(w)
        return layer._adopt(*Q8F.quantizer.quantize(w), linear)


class Q8LinearLora(_QuantLinearBase):
    """Frozen int8 base weight plus a trainable 16-bit low-rank adapter
    (reference: q8_kernels/modules/linear.py:53-113): y = Q8Linear(x) + (x lora_a^T) lora_b^T."""
    weight_dtype = torch.int8

    def __init__(self, in_features: int, out_features: int, r: int, bias: bool = True, device=None,
                 dtype=torch.bfloat16):
        super().__init__(in_features, out_features, bias, device)
        self.r = r
        self.lora_a = nn.Parameter(torch.empty(r, in_features, device=device, dtype=dtype))
        self.lora_b = nn.Parameter(torch.empty(out_features, r, device=device, dtype=dtype))
        nn.init.normal_(self.lora_a, std=1 / r)
        nn.init.zeros_(self.lora_b)

    def forward(self, x, x_scales=None, fuse_gelu=False, out_dtype=None):
        return Q8F.linear.q8_linear_lora(x, self.weight.data, self._bias(), x_scales, self.scales, self.lora_a,
                                         self.lora_b, fuse_gelu, True, out_dtype)

    @classmethod
    def from_linear(cls, linear, r: int, quant_with_hadamard=True):
        if isinstance(linear, Q8Linear):  # share the already quantized weight
            layer = cls(linear.in_features, linear.out_features, r, linear.bias is not None, linear.weight.device)
            layer.weight.data, layer.scales.data = linear.weight.data, linear.scales.data
            if linear.bias is not None:
                layer.bias.data = linear.bias.data
            return layer
        w = linear.weight.data
        assert w.is_cuda, "input linear layer must be in cuda device"
        assert w.dtype == torch.float8_e4m3fn or _is_16bit(w)
        layer = cls(linear.in_features, linear.out_features, r, linear.bias is not None, w.device)
        if quant_with_hadamard:
            w = Q8F.fast_hadamard.hadamard_transform(w)
        return layer._adopt(*Q8F.quantizer.quantize(w), linear)


class FP8Linear(_QuantLinearBase):
    """e4m3 weights with per-output-channel scales; activations are e4m3-quantized per token inside forward."""
    weight_dtype = torch.float8_e4m3fn

    def __init__(self, in_features: int, out_features: int, bias: bool = True, use_hadamard: bool = False, device=None):
        super().__init__(in_features, out_features, bias, device)
        self.use_hadamard = use_hadamard

    def forward(self, x):
        return Q8F.linear.fp8_linear(x, self.weight.data, self._bias(), None, self.scales, self.use_hadamard, x.dtype)

    @classmethod
    def from_linear(cls, linear: nn.Linear, force_cuda=True, use_hadamard=False):
        w = linear.weight.data
        assert w.is_cuda or force_cuda, "input linear layer must be in cuda device"
        assert _is_16bit(w)
        if force_cuda:
            w = w.cuda()
        layer = cls(linear.in_features, linear.out_features, linear.bias is not None, use_hadamard, w.device)
        if use_hadamard:
            w = Q8F.fast_hadamard.hadamard_transform(w)
        layer._adopt(*Q8F.quantizer.quantize_fp8(w), linear)
        if layer.bias is not None:
            layer.bias.data = layer.bias.data.to(w.device)
        return layer

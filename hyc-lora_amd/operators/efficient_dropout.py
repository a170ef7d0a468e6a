"""Dropout that saves no mask: forward and backward regenerate it from a per-module seed and the element index.
Reference: operators/efficient_dropout.py:56-93 (same class names, `apply(x, p, seed)`, a seed drawn once per module,
identity in eval mode, and a backward that masks without rescaling)."""
import torch

from .. import kernels as K


class EfficientMemoryDropoutFunc(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, p, seed):
        ctx.p, ctx.seed = p, seed
        return K.dropout(x.contiguous(), p, seed)

    @staticmethod
    def backward(ctx, grad_out):
        return K.dropout(grad_out.to(torch.bfloat16).contiguous(), ctx.p, ctx.seed, backward=True), None, None


class EfficientMemoryDropout(torch.nn.Module):
    def __init__(self, p):
        super().__init__()
        self.p = p
        self.seed = torch.randint(0, 2 ** 32, (1,)).item()       # one seed per module, fixed for its lifetime

    def forward(self, x):
        if not self.training:
            return x
        return EfficientMemoryDropoutFunc.apply(x, self.p, self.seed)

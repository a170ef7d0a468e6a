"""Gemma's RMSNorm, y = x * rstd * (1 + w), with the input saved compressed.  Reference:
operators/efficient_rmsnorm_gemma.py (identical to efficient_rmsnorm.py but for `w + 1.0` at :59 and :100), so the
kernels are the RMSNorm ones fed with fp32(w) + 1; dw comes back in the weight's dtype."""
from .efficient_rmsnorm import EfficientMemoryRMSNorm, EfficientMemoryRMSNormFunc


class EfficientMemoryRMSNormGemmaFunc(EfficientMemoryRMSNormFunc):
    weight_offset = 1.0


class EfficientMemoryRMSNormGemma(EfficientMemoryRMSNorm):
    _func = EfficientMemoryRMSNormGemmaFunc

"""Swap a model's modules for their memory-efficient counterparts.

Mirrors `replace_module_for_quantization` of the reference's training scripts (train_gsm8k.py:426-592,
train_glue.py:391-493): same selection rules, same constructor keywords taken from the same `compress_config`
sections ("linear", "silu", "layernorm", "softmax", "hadamard", "gemm"), weights re-pointed, recursion into
everything else.  Every kind the reference swaps has a counterpart here.
"""
import torch

from .efficient_dropout import EfficientMemoryDropout
from .efficient_gelu import EfficientMemoryGELU
from .efficient_gemm import EfficientMemoryGEMM, EfficientMemoryGEMMWithSoftmax
from .efficient_hadamard import EfficientMemoryHadamard
from .efficient_layernorm import EfficientMemoryLayerNorm
from .efficient_linear import EfficientMemoryLinear
from .efficient_rmsnorm import EfficientMemoryRMSNorm
from .efficient_rmsnorm_gemma import EfficientMemoryRMSNormGemma
from .efficient_silu import EfficientMemorySiLU
from .efficient_softmax import EfficientMemorySoftmax


def _knobs(section):
    return dict(outlier_ratio=section["outlier_ratio"], sub_outlier_ratio=section["sub_outlier_ratio"],
                rank=section["rank"], sub_outlier_bit=section["sub_outlier_bit"],
                sub_outlier_quantize_method=section["sub_outlier_quant_method"])


def replace_module_for_quantization(module, compress_config, model_args=None, *, mode="ref", group_size=128,
                                    scale_rule="absmax"):
    """In place, like the reference's.  `model_args` is read for `model_name_or_path` only (a name containing "gemma"
    selects the Gemma RMSNorm)."""
    extra = dict(mode=mode, group_size=group_size, scale_rule=scale_rule)
    gemma = model_args is not None and "gemma" in str(getattr(model_args, "model_name_or_path", ""))

    for name, child in module.named_children():
        cls = child.__class__.__name__
        if (isinstance(child, torch.nn.Linear) and child.weight.requires_grad and child.in_features > 100
                and "lm_head" not in name):
            new = EfficientMemoryLinear(in_features=child.in_features, out_features=child.out_features,
                                        bias=child.bias is not None, **_knobs(compress_config["linear"]), **extra)
            new.weight.data = child.weight.data
            if child.bias is not None:
                new.bias.data = child.bias.data
            setattr(module, name, new)
        elif "SiLU" in cls:
            setattr(module, name, EfficientMemorySiLU(**_knobs(compress_config["silu"]), **extra))
        elif "GELU" in cls:
            setattr(module, name, EfficientMemoryGELU(**_knobs(compress_config["silu"]), **extra))   # sic: the "silu" section
        elif "RMSNorm" in cls:
            eps = getattr(child, "variance_epsilon", getattr(child, "eps", 1e-5))
            new = (EfficientMemoryRMSNormGemma if gemma else EfficientMemoryRMSNorm)(normalized_shape=child.weight.data.shape, eps=eps, elementwise_affine=True,
                                         bias=False, **_knobs(compress_config["layernorm"]), **extra)
            new.weight.data = child.weight.data
            setattr(module, name, new)
        elif "LayerNorm" in cls:
            new = EfficientMemoryLayerNorm(normalized_shape=child.weight.data.shape, elementwise_affine=True,
                                           bias=child.bias is not None, **_knobs(compress_config["layernorm"]), **extra)
            new.eps = child.eps                           # (the reference leaves its own default, 1e-5)
            new.weight.data = child.weight.data
            if child.bias is not None:
                new.bias.data = child.bias.data
            setattr(module, name, new)
        elif isinstance(child, torch.nn.Dropout):
            setattr(module, name, EfficientMemoryDropout(0.0))        # sic: the reference swaps in p = 0 (train_gsm8k.py:540-541)
        elif "GEMM" in cls:
            gm = compress_config["gemm"]
            if "gemm1" in name:
                new = EfficientMemoryGEMM(
                    outlier_ratio_1=gm["outlier_ratio"], sub_outlier_ratio_1=gm["sub_outlier_ratio"],
                    sub_outlier_bit_1=gm["sub_outlier_bit"], sub_outlier_quantize_method_1=gm["sub_outlier_quant_method"],
                    outlier_ratio_2=gm["outlier_ratio"], sub_outlier_ratio_2=gm["sub_outlier_ratio"],
                    sub_outlier_bit_2=gm["sub_outlier_bit"], sub_outlier_quantize_method_2=gm["sub_outlier_quant_method"],
                    rank=gm["rank"], **extra)
            else:
                new = EfficientMemoryGEMMWithSoftmax(
                    outlier_ratio_1=compress_config["softmax"]["outlier_ratio"], outlier_ratio_2=gm["outlier_ratio"],
                    sub_outlier_ratio_2=gm["sub_outlier_ratio"], sub_outlier_bit_2=gm["sub_outlier_bit"],
                    sub_outlier_quantize_method_2=gm["sub_outlier_quant_method"], rank=gm["rank"], **extra)
            setattr(module, name, new)
        elif isinstance(child, torch.nn.Softmax):
            setattr(module, name, EfficientMemorySoftmax(outlier_ratio=compress_config["softmax"]["outlier_ratio"]))
        elif "Hadamard" in cls:
            h = compress_config["hadamard"]
            setattr(module, name, EfficientMemoryHadamard(
                outlier_ratio_1=h["outlier_ratio"], sub_outlier_ratio_1=h["sub_outlier_ratio"],
                sub_outlier_bit_1=h["sub_outlier_bit"], sub_outlier_quantize_method_1=h["sub_outlier_quant_method"],
                outlier_ratio_2=h["outlier_ratio"], sub_outlier_ratio_2=h["sub_outlier_ratio"],
                sub_outlier_bit_2=h["sub_outlier_bit"], sub_outlier_quantize_method_2=h["sub_outlier_quant_method"],
                rank=h["rank"], **extra))
        else:
            replace_module_for_quantization(child, compress_config, model_args, mode=mode, group_size=group_size,
                                            scale_rule=scale_rule)

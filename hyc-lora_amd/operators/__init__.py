"""Host-side mirror of the reference's operators/ package: same module, class and function names."""
from . import compress_function, fused_compression  # noqa: F401
from .efficient_gelu import EfficientMemoryGELU, EfficientMemoryGELUFunc  # noqa: F401
from .efficient_hadamard import EfficientMemoryGatedAct, EfficientMemoryHadamard, EfficientMemoryHadamardFunc  # noqa: F401
from .efficient_linear import EfficientMemoryLinear, EfficientMemoryLinearFunc  # noqa: F401
from .efficient_rmsnorm import EfficientMemoryRMSNorm, EfficientMemoryRMSNormFunc  # noqa: F401
from .efficient_silu import EfficientMemorySiLU, EfficientMemorySiLUFunc  # noqa: F401
from .efficient_softmax import EfficientMemorySoftmax, EfficientMemorySoftmaxFunc  # noqa: F401
from .swap import replace_module_for_quantization  # noqa: F401
from .efficient_rmsnorm_gemma import EfficientMemoryRMSNormGemma, EfficientMemoryRMSNormGemmaFunc  # noqa: F401
from .efficient_layernorm import EfficientMemoryLayerNorm, EfficientMemoryLayerNormFunc  # noqa: F401
from .efficient_gemm import (EfficientMemoryGEMM, EfficientMemoryGEMMFunc, EfficientMemoryGEMMWithSoftmax,  # noqa: F401
                             EfficientMemoryGEMMWithSoftmaxFunc)
from ._calibration import calibration_state, load_calibration_state  # noqa: F401
from .efficient_dropout import EfficientMemoryDropout, EfficientMemoryDropoutFunc  # noqa: F401
from .efficient_flashattention import (EfficientFlashAttnVarlenQKVPacked,  # noqa: F401
                                       EfficientFlashAttnVarlenQKVPackedFunc)
